// The evaluator with ONE position per workgroup: four (or eight) wavefronts split the model width.
//
// Quarter q of the width (tiles TW*q .. TW*q+TW-1 of the residual stream, which are also attention
// heads, and a quarter of every matmul's output tiles) belongs to wavefront q, which streams
// exactly the weight blocks of those tiles -- privately, so weights need no cross-wave
// synchronisation.  Quantised activations are exchanged through LDS as ready-made MFMA
// B-operand fragments; row statistics (LayerNorm sums, quantiser maxima) are exchanged as
// per-lane partials and combined in quarter order, which is the group order of the arithmetic
// contract in bf_args.h -- so for the 256-wide network this kernel returns bit for bit what the
// one-wavefront-per-position kernel returns.  The feed-forward block runs in steps of 512 hidden
// channels: each quarter computes four hidden tiles per step, so a 256-wide quantiser chunk spans
// a pair of quarters and its maximum is exchanged; the float64 sums over the chunks stay in order.
//
// Three forms, selected by TWIN and OCTO, with identical results:
//   TWIN = false  one workgroup per compute unit, 512 registers per wave.  Weight blocks stream
//                 through a private LDS ring per wave (direct-to-LDS loads, SLOTS blocks deep),
//                 attention is software-pipelined across heads.
//   TWIN = true   two workgroups per compute unit: at most 80 KiB of LDS and 256 registers per
//                 wave, so every SIMD holds two wavefronts of different positions and one's
//                 waits (LDS round trips, barriers, MFMA results) are covered by the other's
//                 work.  Weight fragments go from L2 straight to registers (half a block = four
//                 fragments at a time, prefetched through a rotation of register sets).
//                 Highest throughput.
//   OCTO          (with TWIN's register weight path) eight wavefronts per position, one workgroup
//                 per compute unit: a quarter belongs to two wavefronts, `sub` = 0 and 1, each
//                 owning half of the quarter's tiles in every matmul and reading its blocks out
//                 of the quarter's stream where they lie (block_at).  A quarter's LayerNorm chain
//                 is started by its first wavefront and continued by its second.  Lowest latency
//                 per position (launches of up to one position per compute unit).
//
// LDS map (bytes): [ring: 4 waves x SLOTS x 8 KiB, absent in the TWIN form] [xch: 3 slots of
// 64 floats per wave] [hid: the whole quantised hidden row (32 KiB at width 256, 64 KiB at width
// 512 with eight wavefronts) or one step of it (16 KiB: width 512 with the weight ring)]
// [act: NT KiB] [par: one copy of each quarter's side parameters -- the wave's own with four
// wavefronts, shared by the quarter's two with eight].  During the heads the normalised stream
// (NT*4 KiB, fp32) overlays hid/act/par.
#pragma once

#include <atomic>

#include "bf_device.hip.h"

// TWIN form: workgroups per compute unit, and register sets of the weight prefetch (one set =
// half a block; SETS - 1 half-blocks are in flight).  Measured on MI355X at batch 4096: three
// workgroups per unit spill too much (81-103 registers); three sets run without a spill
// (1.717 ms), four spill 8 registers (1.741 ms), six 61 (2.10 ms).
#ifndef BF_TWIN_SETS
#define BF_TWIN_SETS 3
#endif
#ifndef BF_TWIN_OCC
#define BF_TWIN_OCC 2
#endif
// Eight-wavefront form: register sets of its weight prefetch.  Measured: 256-wide network, 64
// positions: 0.136 ms with four sets, 0.137 with three, 0.138 with six; 512-wide network, 4096
// positions: 12.5 ms with four, 12.8 with three, 16.0 with six (68 spilled registers).
#ifndef BF_TWIN_AHEAD_FFN
#define BF_TWIN_AHEAD_FFN 1
#endif
#ifndef BF_BIASED_ACC
#define BF_BIASED_ACC 1
#endif
#ifndef BF_FORCE_ACTL
#define BF_FORCE_ACTL 0
#endif
#ifndef BF_OCTO_SETS
#define BF_OCTO_SETS 4
#endif

// Timing experiments (BF_EXP_*): compile-time switches that replace a part of a kernel by a
// cheaper stand-in to measure what that part costs.  Their results are wrong by construction, so
// they compile only together with BF_TIMING_BUILD, which the library's own build never defines
// (brokefish_amd/_build.py refuses both).
#if (defined(BF_EXP_NOF32) || defined(BF_EXP_NOMFMA) || defined(BF_EXP_SAMEBLOCK) || defined(BF_EXP_NOLOAD) || \
     defined(BF_EXP_HALFLOAD) || defined(BF_EXP_NOBARRIER) || defined(BF_EXP_SAMELAYER) || defined(BF_EXP_NOWARM)) && !defined(BF_TIMING_BUILD)
#error "BF_EXP_* switches give wrong results: they need BF_TIMING_BUILD and never go into the library"
#endif
#ifdef BF_EXP_NOF32   // timing experiment: one vector instruction in place of an fp32 matrix step
#define BF_F32MMA(a_, b_, c_) ([&]() { v16f r_ = (c_); r_[0] = __builtin_fmaf((a_), (b_), r_[0]); return r_; }())
#else
#define BF_F32MMA(a_, b_, c_) __builtin_amdgcn_mfma_f32_32x32x2f32((a_), (b_), (c_), 0, 0, 0)
#endif

namespace bf {
namespace board {

extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

template <int DM, bool TWIN, bool OCTO = false>
struct Cfg : Layout<DM> {
    typedef Layout<DM> L;
    static constexpr int NW = OCTO ? 8 : 4;   // wavefronts per position
    static constexpr int RING_BYTES = TWIN ? 0 : 4 * L::SLOTS * BLOCK;
    static constexpr int XCH_OFF = RING_BYTES;
    static constexpr int HID_OFF = XCH_OFF + 3 * (NW / 4) * FRAG;
    // the quantised hidden row of the feed-forward block: the whole row (F / 32 tiles) where it fits
    // -- the 256-wide network (32 KiB), and the 512-wide one (64 KiB) with eight wavefronts, no
    // weight ring and one parameter copy per quarter; otherwise one step of 512 channels (16 tiles)
    static constexpr bool FULLHID = DM == 256 || (OCTO && DM == 512);
    static constexpr int HID_FRAGS = FULLHID ? L::F / 32 : 16;
    static constexpr int ACT_OFF = HID_OFF + HID_FRAGS * FRAG;
    static constexpr int PAR_OFF = ACT_OFF + L::NT * FRAG;
    // three workgroups per compute unit: only the often-read part of the feed-forward parameters
    // is kept in LDS, the rest is read from global memory where it is used
    static constexpr bool BTAIL_GLOBAL = TWIN && !OCTO && BF_TWIN_OCC >= 3;
    static constexpr int PWL_FLOATS = L::A_FLOATS + (BTAIL_GLOBAL ? L::B_LDS_FLOATS : L::B_FLOATS);   // per copy, in LDS
    // four wavefronts: every wave keeps its own copy of its quarter's parameters (no wave waits for
    // another's transfer).  Eight: the two waves of a quarter share one copy, fetched by the first.
    static constexpr int PAR_COPIES = 4;
    static constexpr int LDS_BYTES = PAR_OFF + PAR_COPIES * PWL_FLOATS * 4;
    static_assert(!OCTO || TWIN, "eight wavefronts per position take their weights straight to registers");
    static_assert(LDS_BYTES <= (TWIN && !OCTO ? 160 / BF_TWIN_OCC : 160) * 1024, "LDS budget: one or two workgroups per compute unit");
    static_assert(L::NT * 4 * FRAG <= LDS_BYTES - HID_OFF, "normalised stream overlay");
    static_assert(L::BPW % L::SLOTS == 0, "ring slot of a block must not depend on the layer");
    static_assert((2 * L::BPW) % BF_TWIN_SETS == 0, "register set of a half-block must not depend on the layer");
};

// workgroup barrier that waits for this wave's LDS traffic only (outstanding direct-to-LDS
// weight loads stay in flight)
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// bytes (a multiple of 16) from global to LDS without passing through registers
__device__ __forceinline__ void dma(const float* src, float* dst, int nfloats, int lane) {
    const uint8_t* s = reinterpret_cast<const uint8_t*>(src) + lane * 16;
    uint8_t* d = reinterpret_cast<uint8_t*>(dst);
    const int bytes = nfloats * 4, full = bytes / FRAG, rem = (bytes % FRAG) / 16;
    for (int i = 0; i < full; i++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(s + i * FRAG),
                                         (__attribute__((address_space(3))) void*)(d + i * FRAG), 16, 0, 0);
    if (lane < rem)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(s + full * FRAG),
                                         (__attribute__((address_space(3))) void*)(d + full * FRAG), 16, 0, 0);
}

// one 16-byte fragment step of a block product: a 32-deep int8 MFMA, or two 16-deep e4m3 steps
template <bool SWAP>
__device__ __forceinline__ v16i frag_mma(const v4i& w, const v4i& act, const v16i& acc) {
#ifdef BF_EXP_NOMFMA   // timing experiment: one vector instruction in place of the product
    v16i r = acc;
    r[0] += w[0] ^ act[0];
    return r;
#endif
    return SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(act, w, acc, 0, 0, 0)
                : __builtin_amdgcn_mfma_i32_32x32x32_i8(w, act, acc, 0, 0, 0);
}
template <bool SWAP>
__device__ __forceinline__ v16f frag_mma(const v4i& w, const v4i& act, v16f acc) {
    const v2l wl = __builtin_bit_cast(v2l, w), al = __builtin_bit_cast(v2l, act);
#pragma unroll
    for (int h = 0; h < 2; h++) acc = e4m3_step<SWAP>(wl[h], al[h], acc);
    return acc;
}

// acc * sa summed over the k-chunks in float64, cast once (one chunk: the fp32 product, which
// is the same number).  BIASED: the int32 accumulator started at the bit pattern of 1.5 * 2^23,
// so its bits read as a float are 1.5 * 2^23 + acc exactly (|acc| <= 127 * 127 * 256 < 2^22) and
// one fp32 subtraction, which is exact, replaces the slower integer-to-float conversion.
constexpr int ACC_BIAS_BITS = 0x4b400000;
constexpr float ACC_BIAS = 12582912.0f;
template <int KC, bool BIASED, typename ACC>
__device__ __forceinline__ float chunk_sum(const ACC (&acc)[KC], int i, const float (&sa)[KC]) {
    if constexpr (KC == 1) {
        if constexpr (BIASED) return (__int_as_float(acc[0][i]) - ACC_BIAS) * sa[0];
        else return accf(acc[0], i) * sa[0];
    } else {
        static_assert(!BIASED, "the biased accumulator is used with a single k-chunk");
        double o = (double)acc[0][i] * (double)sa[0];
#pragma unroll
        for (int c = 1; c < KC; c++) o = __builtin_fma((double)acc[c][i], (double)sa[c], o);
        return (float)o;
    }
}
// the accumulator's value as the debug taps report it
template <bool BIASED>
__device__ __forceinline__ int tapbits(const v16i& a, int i) { return BIASED ? a[i] - ACC_BIAS_BITS : a[i]; }
template <bool BIASED>
__device__ __forceinline__ int tapbits(const v16f& a, int i) { return __float_as_int(a[i]); }

// Position of a wave's n-th weight block of a layer inside its quarter's stream: a + sub * b.
// With four wavefronts per position a wave consumes its quarter's stream in order (a = n).  With
// eight, the two wavefronts of a quarter (sub = 0, 1) each take half of the quarter's tiles in
// every matmul, so a wave's blocks are every other group of the same stream.
struct BlockAt { int a, b; };
template <int KC, int TW, int SUB, bool FULLHID>
__host__ __device__ constexpr BlockAt block_at(int n) {
    constexpr int TWW = TW / SUB, HT = 4 / SUB;
    constexpr int NQ = 3 * KC * TWW, NO = KC * TWW, SSTR = 4 * KC + 2 * TW, BASE = 4 * KC * TW;
    if (n < NQ) return {3 * KC * (n / (3 * KC)) + n % (3 * KC), 3 * KC * TWW};
    if (n < NQ + NO) return {3 * KC * TW + KC * ((n - NQ) / KC) + (n - NQ) % KC, KC * TWW};
    const int m = n - NQ - NO;
    if constexpr (!FULLHID) {
        // step by step: the step's hidden tiles, then its two k-chunks of the second matmul
        constexpr int SW_ = HT * KC + 2 * TWW;
        const int st = m / SW_, r = m % SW_, base = BASE + st * SSTR;
        if (r < HT * KC) return {base + KC * (r / KC) + r % KC, KC * HT};
        return {base + 4 * KC + ((r - HT * KC) / TWW) * TW + (r - HT * KC) % TWW, TWW};
    } else {
        // every step's hidden tiles first, then the second matmul tile by tile over all k-chunks
        // (the stream keeps the step-by-step order; chunk cc lies in step cc / 2)
        constexpr int STEPS = TW, KCF = 2 * STEPS, NF1 = STEPS * HT * KC;
        if (m < NF1) return {BASE + (m / (HT * KC)) * SSTR + m % (HT * KC), KC * HT};
        const int i = (m - NF1) / KCF, cc = (m - NF1) % KCF;
        return {BASE + (cc / 2) * SSTR + 4 * KC + (cc % 2) * TW + i, TWW};
    }
}

// Every wave's block sequence of a layer stays inside the layer's BPW blocks and the waves of a
// quarter together visit each block exactly once (so no prefetch address leaves the stream: the
// sequence only ever continues into the following layer or the head blocks).
template <int KC, int TW, int SUB, int BPW, bool FULLHID>
constexpr bool block_at_covers_layer() {
    bool seen[BPW] = {};
    for (int sub = 0; sub < SUB; sub++)
        for (int n = 0; n < BPW / SUB; n++) {
            const BlockAt at = block_at<KC, TW, SUB, FULLHID>(n);
            const int i = at.a + sub * at.b;
            if (i < 0 || i >= BPW || seen[i]) return false;
            seen[i] = true;
        }
    return true;
}

template <int DM, bool TAPS, bool TWIN, bool FP8, bool OCTO = false, bool PROF = false>
__global__ __launch_bounds__(OCTO ? 2 * THREADS : THREADS, TWIN && !OCTO ? BF_TWIN_OCC : 1) void board_kernel(const KArgs a) {
    typedef Cfg<DM, TWIN, OCTO> C;
    typedef typename Acc<FP8>::type acc_t;
    static_assert(!FP8 || DM == 256, "e4m3: one k-chunk per matmul of the width (fp32 sums over the chunks of ffn2 only)");
    constexpr int D = C::D, F = C::F, NT = C::NT, TW = C::TW, CW = C::CW, KC = C::KC, KCF = C::KCF;
    constexpr int STEPS = C::STEPS, BPW = C::BPW, HB = C::HB, SLOTS = C::SLOTS, WPC = 4 / KC;
    constexpr int NW = C::NW, SUB = NW / 4;   // wavefronts per position; wavefronts sharing a quarter of the width
    constexpr int TWW = TW / SUB;             // tiles of the width a wave owns
    constexpr int HT = 4 / SUB;               // hidden tiles a wave computes per feed-forward step
    constexpr int NB = BPW / SUB;             // weight blocks a wave consumes per layer
    // register sets of the prefetch: NSETS - 1 half-blocks in flight
    // (the 512-wide network's eight-wave form: three sets measure the same as four and spill
    // 15 registers instead of 26)
    constexpr int NSETS = OCTO ? (DM == 512 ? 3 : BF_OCTO_SETS) : BF_TWIN_SETS;
    static_assert(TW % SUB == 0 && (2 * NB) % NSETS == 0, "tiles and register sets must split evenly");
    constexpr bool FULLHID = C::FULLHID;      // the whole quantised hidden row stays in LDS
    static_assert(block_at_covers_layer<KC, TW, SUB, BPW, FULLHID>(), "block_at must enumerate a layer's blocks exactly once");
    static_assert(!FULLHID || (STEPS == TW && KCF == 2 * STEPS), "the full-row form: as many steps as tiles per quarter, two k-chunks per step");
    static_assert(SLOTS <= HB && NSETS - 1 <= 2 * HB + 2, "the first prefetches of a heads-only run stay inside the head blocks");
    constexpr int XS = NW * 64;               // floats of one exchange slot
    // Eight wavefronts on the 512-wide network: a wave has 256 registers and the quantised row alone
    // would take 64 of them, so the activation fragments are read from LDS at each MFMA instead.
    constexpr bool ACTL = (OCTO && DM == 512) || BF_FORCE_ACTL;
    // One wave per SIMD (!TWIN, 512 registers): a tile's product is issued before the previous
    // tile's epilogue, and Q, K and V together, so the matrix pipe works under the vector work of
    // the same wave.  Two waves per SIMD (256 registers each): one product at a time, issued after
    // the previous epilogue -- the second set of accumulators would spill, and the SIMD's other
    // wave fills the gap.  Measured at batch 4096 (TWIN): 1.72 ms without a spill, against
    // 1.90 ms with 20 spilled registers when issuing ahead.
    // int8 with one k-chunk per matmul of the width: the QKV, out-projection and first
    // feed-forward accumulators start at the bit pattern of 1.5 * 2^23 (see chunk_sum), held in
    // 16 registers that every such product reads as its addend.
    constexpr bool BIASED = !FP8 && KC == 1 && BF_BIASED_ACC;
    constexpr bool AHEAD = !TWIN;
    // In the feed-forward block of the full-row form the register file has room for the second
    // accumulator at two waves per SIMD as well (only one tile's sums over the chunks are alive).
    constexpr bool AH_FFN = AHEAD || (FULLHID && BF_TWIN_AHEAD_FFN);
    constexpr int HALF = BLOCK / 2;   // four fragments: the unit of the register prefetch (TWIN)
    constexpr int VM_AHEAD = TAPS ? 0 : (SLOTS - 1) * 8;   // ring loads that may stay in flight at a ring wait
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = OCTO ? (wave & 3) : wave;   // the quarter of the width this wave works in
    const int sub = OCTO ? (wave >> 2) : 0;   // which of the quarter's waves it is
    const int t0 = TWW * sub, h0 = HT * sub;  // its first tile of the quarter, its first hidden tile of a step
    const int t = lane & 31, g = lane >> 5;
    // the position this workgroup evaluates: its own number, or entry blockIdx.x of the compacted
    // leaf list; a skipped position / a slot past the list's count: the whole workgroup leaves
    // before any barrier
    int b = blockIdx.x;
    if (a.leaf_index) {
        if (b >= *a.leaf_count) return;
        b = __builtin_amdgcn_readfirstlane(a.leaf_index[b]);
        if ((unsigned)b >= (unsigned)a.n) return;   // not a position of this launch
    }
    if (a.active && !a.active[b]) return;
    const int nl_run = a.l1 - a.l0;
    // Phase accounting (PROF builds only): the shader clock is read at phase boundaries and the
    // cycles since the previous mark are charged to a slot; the time spent inside workgroup
    // barriers is summed separately (and is also contained in the enclosing phases).
    unsigned long long ph[N_PHASES];
    unsigned long long t_mark = 0, t_begin = 0, t_sync = 0;
    if constexpr (PROF) {
#pragma unroll
        for (int i = 0; i < N_PHASES; i++) ph[i] = 0;
        t_mark = t_begin = __builtin_readcyclecounter();
    }
#define BF_PHASE(slot)                                                    \
    do {                                                                  \
        if constexpr (PROF) {                                             \
            __builtin_amdgcn_sched_barrier(0); /* nothing is scheduled across the mark */ \
            const unsigned long long now_ = __builtin_readcyclecounter(); \
            __builtin_amdgcn_sched_barrier(0);                            \
            ph[slot] += now_ - t_mark;                                    \
            t_mark = now_;                                                \
        }                                                                 \
    } while (0)
    auto barrier = [&]() {
        if constexpr (PROF) {
            const unsigned long long t0_ = __builtin_readcyclecounter();
            lds_barrier();
            t_sync += __builtin_readcyclecounter() - t0_;
        } else {
            lds_barrier();
        }
    };

    uint8_t* const myring = lds + wave * (SLOTS * BLOCK);   // !TWIN
    float* const xch = reinterpret_cast<float*>(lds + C::XCH_OFF);
    uint8_t* const hid = lds + C::HID_OFF;
    uint8_t* const act = lds + C::ACT_OFF;
    // the quarter's side parameters in LDS: with four waves the wave's own copy; with eight one copy
    // per quarter, transferred by the quarter's first wave at points where a workgroup barrier
    // separates the transfer from the other wave's last read of the old and first read of the new
    constexpr bool SHARED_PAR = OCTO;
    const bool par_owner = !SHARED_PAR || sub == 0;
    float* const pA = reinterpret_cast<float*>(lds + C::PAR_OFF) + q * C::PWL_FLOATS;
    constexpr int B_COPY = C::BTAIL_GLOBAL ? C::B_LDS_FLOATS : C::B_FLOATS;
    float* const pB = pA + C::A_FLOATS;
    // the quarter's weight stream, from the first layer that runs; block `seq` in the quarter's order
    const uint8_t* const wsrc =
        a.wstream + ((size_t)q * ((size_t)a.n_layers * BPW + HB + 1) + (size_t)a.l0 * BPW) * BLOCK + lane * 16;
    const float* const wpar = a.fparams + (size_t)q * a.n_layers * C::PW_FLOATS;   // the quarter's [layer][PW]
    const float* const gp = a.fparams + (size_t)4 * a.n_layers * C::PW_FLOATS;       // tables, final norm

    // TWIN: half-block `hseq` of this wave's stream (consumption order) into register set `set`
    v4i frt[NSETS][4];
    auto load_half = [&](int hseq, int set) {
#ifdef BF_EXP_SAMEBLOCK   // timing experiment: every weight load hits the same 4 KiB (L1 hits)
        const uint8_t* src = wsrc + (size_t)(hseq & 1) * HALF;
#else
        const uint8_t* src = wsrc + (size_t)hseq * HALF;
#endif
#ifdef BF_EXP_NOLOAD   // timing experiment: no weight traffic
        (void)src;
#pragma unroll
        for (int s = 0; s < 4; s++) asm volatile("" : "=v"(frt[set][s]));
#elif defined(BF_EXP_HALFLOAD)   // timing experiment: half of the weight traffic
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (s & 1) asm volatile("" : "=v"(frt[set][s]));
            else frt[set][s] = *reinterpret_cast<const v4i*>(src + s * FRAG);
        }
#else
#pragma unroll
        for (int s = 0; s < 4; s++) frt[set][s] = *reinterpret_cast<const v4i*>(src + s * FRAG);
#endif
    };
    // the wave's hh-th half-block of the layer whose stream starts at block `base` (hh may run into
    // the following layer, whose stream starts at block `next`) into its register set
    auto fetch_half = [&](int hh, int base, int next) {
        const int n = hh / 2;
        const BlockAt at = block_at<KC, TW, SUB, FULLHID>(n % NB);
        load_half(2 * ((n < NB ? base : next) + at.a + sub * at.b) + hh % 2, hh % NSETS);
    };
    // !TWIN: block `seq` into ring slot `slot`; a slot into the fragment registers
    v4i fr[8];
    auto issue_block = [&](int seq, int slot) {
        const uint8_t* src = wsrc + (size_t)seq * BLOCK;
        uint8_t* dst = myring + slot * BLOCK;
#pragma unroll
        for (int s = 0; s < 8; s++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + s * FRAG),
                                             (__attribute__((address_space(3))) void*)(dst + s * FRAG), 16, 0, 0);
    };
    auto read_slot = [&](int slot) {
#pragma unroll
        for (int s = 0; s < 8; s++) fr[s] = *reinterpret_cast<const v4i*>(&myring[slot * BLOCK + s * FRAG + lane * 16]);
    };
    // Row sum over the width.  Every tile's 16 values form one chain from zero; a wave adds the sums
    // of its own tiles as a balanced tree and publishes the result; with eight waves the two halves
    // of a quarter are added, then the four quarter sums in order -- the same tree whichever way
    // the width is split over waves.  One exchange slot per call site (`slot`), so that a fast
    // wave's next partial cannot overwrite what a slow wave still reads: between two uses of a
    // slot lies at least one other workgroup barrier.
    auto tiles_sum = [&](const float (&ts)[TWW]) -> float {
        static_assert(TWW == 1 || TWW == 2 || TWW == 4, "tile sums are added as a balanced tree");
        if constexpr (TWW == 1) return ts[0];
        else if constexpr (TWW == 2) return ts[0] + ts[1];
        else return (ts[0] + ts[1]) + (ts[2] + ts[3]);
    };
    auto xsum = [&](float part, int slot) -> float {
        xch[slot * XS + wave * 64 + lane] = part;
        barrier();
        const float* p = xch + slot * XS + lane;
        if constexpr (!OCTO) return ((p[0] + p[64]) + p[128]) + p[192];
        else return (((p[0] + p[256]) + (p[64] + p[320])) + (p[128] + p[384])) + (p[192] + p[448]);
    };
    // LayerNorm of this wave's channels; gamma / beta point at this wave's slice
    auto layernorm = [&](const float (&x)[TWW][16], const float* gamma, const float* beta, float (&y)[TWW][16]) {
        float ts[TWW];
#pragma unroll
        for (int i = 0; i < TWW; i++) {
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) acc = acc + x[i][r];
            ts[i] = acc;
        }
        const float s = xsum(tiles_sum(ts), 0);
        const float mean = (s + partner(s, g)) * (1.0f / D);
#pragma unroll
        for (int i = 0; i < TWW; i++) {
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float d = x[i][r] - mean;
                acc = __builtin_fmaf(d, d, acc);
            }
            ts[i] = acc;
        }
        const float v = xsum(tiles_sum(ts), 1);
        const float var = (v + partner(v, g)) * (1.0f / D);
        const float rstd = 1.0f / __builtin_sqrtf(var + a.eps);
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f ga = ldg4(gamma + 32 * i + 8 * j + 4 * g);
                const v4f be = ldg4(beta + 32 * i + 8 * j + 4 * g);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float d = x[i][4 * j + k] - mean;
                    y[i][4 * j + k] = __builtin_fmaf(d * rstd, ga[k], be[k]);
                }
            }
    };
    // signed quantiser of a row spread over the four waves: per 256-wide chunk one scale; this
    // wave's bytes go to the activation buffer, every wave then reads the whole row back
    auto quant_exchange = [&](const float (&y)[TWW][16], float (&sa)[KC], v4i (&qv)[NT], int8_t* tap, size_t tap_row) {
        float am = 0.0f;
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) am = __builtin_fmaxf(am, __builtin_fabsf(y[i][r]));
        xch[2 * XS + wave * 64 + lane] = am;
        barrier();
#pragma unroll
        for (int c = 0; c < KC; c++) {
            float m = 0.0f;   // the maximum is exact in any order: every wave of the chunk's quarters
#pragma unroll
            for (int w = c * WPC; w < (c + 1) * WPC; w++)
#pragma unroll
                for (int u = 0; u < SUB; u++) m = __builtin_fmaxf(m, xch[2 * XS + (w + 4 * u) * 64 + lane]);
            m = __builtin_fmaxf(m, partner(m, g));
            sa[c] = m > 0.0f ? (FP8 ? m * 0.125f : div127(m)) : 1.0f;
        }
        const float so = KC == 1 ? sa[0] : (q < WPC ? sa[0] : sa[KC - 1]);
        const float inv = 1.0f / so;
#pragma unroll
        for (int i = 0; i < TWW; i++) {
            v4i w;
#pragma unroll
            for (int j = 0; j < 4; j++)
                w[j] = (int)quant4<FP8>(y[i][4 * j], y[i][4 * j + 1], y[i][4 * j + 2], y[i][4 * j + 3], so, inv);
            *reinterpret_cast<v4i*>(act + (TW * q + t0 + i) * FRAG + lane * 16) = w;
            if (TAPS && tap)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(tap + (tap_row * T + t) * D + 32 * (TW * q + t0 + i) + 8 * j + 4 * g) = w[j];
        }
        barrier();
        if constexpr (!ACTL)
#pragma unroll
            for (int n = 0; n < NT; n++) qv[n] = *reinterpret_cast<const v4i*>(act + n * FRAG + lane * 16);
    };
    // where a block product takes its eight activation fragments from: registers, or (ACTL) LDS
    struct FragSrc { const v4i* reg; const uint8_t* mem; };
    auto fragments = [&](const v4i* regs, const uint8_t* buf, int first) -> FragSrc {
        return FragSrc{regs + first, buf + first * FRAG + lane * 16};
    };
    auto fragment = [&](const FragSrc& f, int s) -> v4i {
        if constexpr (ACTL) return *reinterpret_cast<const v4i*>(f.mem + s * FRAG);
        else return f.reg[s];
    };

    acc_t acc_start = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (BIASED)
#pragma unroll
        for (int r = 0; r < 16; r++) {   // opaque to the compiler, so the vector stays in registers
            int m;
            asm volatile("v_mov_b32 %0, 0x4b400000" : "=v"(m));
            acc_start[r] = m;
        }

    // ---- start the weight stream and the first layer's parameters ------------------------------
    if constexpr (TWIN) {
        // a run of no layers (heads only) starts at the head blocks, which block_at does not
        // describe: the stream is started below, where the heads restart it
        if (nl_run > 0)
#pragma unroll
            for (int j = 0; j < NSETS - 1; j++) fetch_half(j, 0, BPW);
    } else {
#pragma unroll
        for (int j = 0; j < SLOTS; j++) issue_block(j, j);   // layer blocks, or the first head blocks (SLOTS <= HB)
    }
    if (nl_run > 0 && par_owner) {
        dma(wpar + (size_t)a.l0 * C::PW_FLOATS, pA, C::A_FLOATS, lane);
        dma(wpar + (size_t)a.l0 * C::PW_FLOATS + C::A_FLOATS, pB, B_COPY, lane);
    }

    // ---- embedding (this wave's channels) --------------------------------------------------------
    float x[TWW][16];
    // An encoder-only launch (tap table with `alive`): the residual stream comes in through x_in, the
    // token mask through `alive`, the stream after the last layer goes out through resid_last, and
    // there are no board words and no heads.
    const bool enc_only = TAPS && a.taps.alive != nullptr;
    const unsigned word = enc_only ? (a.taps.alive[(size_t)b * T + t] ? 0u : 0x800u) : a.boards[(size_t)b * T + t];
    const int ctrl = enc_only ? 1 : a.control[b];
    const unsigned alive = (unsigned)__ballot(((word >> 11) & 1) == 0 && g == 0);
    if (TAPS && a.taps.x_in) {
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = ldg4(a.taps.x_in + ((size_t)b * T + t) * D + 32 * (TW * q + t0 + i) + 8 * j + 4 * g);
#pragma unroll
                for (int k = 0; k < 4; k++) x[i][4 * j + k] = v[k];
            }
    } else {
        const int stm = ctrl < 0;
        int clock = (ctrl < 0 ? -ctrl : ctrl) - 1;
        clock = clock < 0 ? 0 : (clock > 100 ? 100 : clock);
        int rp = a.rep[b];
        rp = rp > 2 ? 2 : rp;
        int ts = ((word >> 6) & 7) * 2 + ((word >> 9) & 1);
        ts = ts > 11 ? 11 : ts;
        const int ct = ((word >> 10) & 1) * 2 + stm;
        const int own = CW * q + 32 * t0 + 4 * g;
        const float* e_sq = gp + C::G_SQ + (word & 63) * D + own;
        const float* e_ts = gp + C::G_TS + ts * D + own;
        const float* e_ct = gp + C::G_CT + ct * D + own;
        const float* e_ck = gp + C::G_CLOCK + clock * D + own;
        const float* e_rp = gp + C::G_REP + rp * D + own;
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = 32 * i + 8 * j;
                const v4f vs = ldg4(e_sq + c), vt = ldg4(e_ts + c), vc = ldg4(e_ct + c);
                const v4f vk = ldg4(e_ck + c), vr = ldg4(e_rp + c);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float per_board = vk[k] + vr[k];
                    float v = vs[k] + vt[k];
                    v = v + vc[k];
                    x[i][4 * j + k] = v + per_board;
                }
            }
    }
    if (TAPS && a.taps.embed)
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.embed[((size_t)b * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = x[i][r];

    wait_vm<0>();   // the parameters (and the first ring slots) have landed
    if constexpr (!TWIN) read_slot(0);
    BF_PHASE(PH_EMBED);

    for (int l = a.l0; l < a.l1; l++) {
        const int li = l - a.l0;
        const size_t bl = (size_t)b * nl_run + li;   // tap row
        const int lnext = l + 1 < a.l1 ? l + 1 : l;  // after the last layer the same slice is fetched again
        // the rarely read tail of the feed-forward parameters: in LDS with the rest, or in global memory
        const float* const pBt = C::BTAIL_GLOBAL ? wpar + (size_t)l * C::PW_FLOATS + C::A_FLOATS : pB;
        // Multiply by the wave's k-th block of this layer (its own count: see block_at).
        // TWIN: its two halves sit in register sets 2k % NSETS and (2k + 1) % NSETS; a set is refilled
        // with the wave's half-block NSETS positions on once it has been consumed.  Four waves: that
        // runs on into the next layer and, after the last one, into the head blocks.  Eight waves:
        // after the last layer of the run the same layer is fetched again (and never used).
        // !TWIN: the block is in `fr`; the ring slot it came from is refilled SLOTS blocks ahead,
        // then block k+1 is read from its slot.
        const int lbase = li * BPW, lfollow = OCTO ? (lnext - a.l0) * BPW : (li + 1) * BPW;
#define BF_WMM(SWAP, k, actp) BF_WMM_FROM(SWAP, k, actp, acc_start)
#define BF_WMM_FROM(SWAP, k, actp, init)                                                             \
    ([&]() -> acc_t {                                                                                \
        const FragSrc act_ = (actp);                                                                 \
        acc_t r_ = (init);                                                                           \
        if constexpr (TWIN) {                                                                        \
            fetch_half(2 * (k) + NSETS - 1, lbase, lfollow);                                         \
            _Pragma("unroll") for (int s_ = 0; s_ < 4; s_++)                                         \
                r_ = frag_mma<SWAP>(frt[(2 * (k)) % NSETS][s_], fragment(act_, s_), r_);             \
            fetch_half(2 * (k) + NSETS, lbase, lfollow);                                             \
            _Pragma("unroll") for (int s_ = 0; s_ < 4; s_++)                                         \
                r_ = frag_mma<SWAP>(frt[(2 * (k) + 1) % NSETS][s_], fragment(act_, 4 + s_), r_);     \
        } else {                                                                                     \
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                       \
            issue_block(((k) + SLOTS < NB ? lbase : lfollow) + block_at<KC, TW, 1, FULLHID>(((k) + SLOTS) % NB).a, (k) % SLOTS); \
            _Pragma("unroll") for (int s_ = 0; s_ < 8; s_++)                                         \
                r_ = frag_mma<SWAP>(fr[s_], fragment(act_, s_), r_);                                 \
            wait_vm<VM_AHEAD>();                                                                     \
            read_slot(((k) + 1) % SLOTS);                                                            \
        }                                                                                            \
        return r_;                                                                                   \
    }())

        // ---- LayerNorm 1, quantise, exchange ----------------------------------------------------------
        v4i xq[NT];
        float sa[KC];
        {
            float y[TWW][16];
            layernorm(x, pA + C::A_LN1G + 32 * t0, pA + C::A_LN1B + 32 * t0, y);
            quant_exchange(y, sa, xq, TAPS ? a.taps.qa_qkv : nullptr, bl);
        }
        // a shared copy's feed-forward parameters of this layer (the first layer's came with the start)
        if (SHARED_PAR && par_owner && li > 0) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)l * C::PW_FLOATS + C::A_FLOATS, pB, B_COPY, lane);
        }
        BF_PHASE(PH_LN1);
        float sa_tok[KC][16];   // activation scale of token ch(r, g), for the V tiles whose rows are tokens
        if constexpr (AHEAD)
#pragma unroll
            for (int c = 0; c < KC; c++)
#pragma unroll
                for (int r = 0; r < 16; r++) sa_tok[c][r] = __shfl(sa[c], ch(r, g));

        // ---- attention over this wave's heads ----------------------------------------------------------
        // !TWIN: software-pipelined -- the three weight GEMMs of head i+1 are issued right after the
        // score MFMAs of head i, so the matrix pipe works through them under head i's softmax.
        float o[TWW][16];
        acc_t accq[KC], acck[KC], accv[KC];
#pragma unroll
        for (int i = 0; i < TWW; i++) {
            if (AHEAD && i == 0) {
#pragma unroll
                for (int c = 0; c < KC; c++) accq[c] = BF_WMM(false, 3 * KC * i + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int c = 0; c < KC; c++) acck[c] = BF_WMM(false, 3 * KC * i + KC + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int c = 0; c < KC; c++) accv[c] = BF_WMM(true, 3 * KC * i + 2 * KC + c, fragments(xq, act, 8 * c));
            }
            const int h = TW * q + t0 + i;
            float qf[16], kf[16], vf[16];
            {
                const int ti = t0 + i;   // this head's tile within the quarter
                const float swq = pA[C::A_SW + ti], swk = pA[C::A_SW + TW + ti], swv = pA[C::A_SW + 2 * TW + ti];
                const float bv = pA[C::A_BV + 32 * ti + t];
                v4f bq[4], bk[4];
                load_tile16(pA + C::A_BQ + 32 * ti, g, bq);
                load_tile16(pA + C::A_BK + 32 * ti, g, bk);
                // !AHEAD: one product at a time, descaled before the next one starts
                if constexpr (!AHEAD)
#pragma unroll
                    for (int c = 0; c < KC; c++) accq[c] = BF_WMM(false, 3 * KC * i + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) qf[4 * j + k] = chunk_sum<KC, BIASED>(accq, 4 * j + k, sa) * swq + bq[j][k];
                if constexpr (!AHEAD) {
                    pin16(qf);
#pragma unroll
                    for (int c = 0; c < KC; c++) acck[c] = BF_WMM(false, 3 * KC * i + KC + c, fragments(xq, act, 8 * c));
                }
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) kf[4 * j + k] = chunk_sum<KC, BIASED>(acck, 4 * j + k, sa) * swk + bk[j][k];
                if constexpr (!AHEAD) {
                    pin16(kf);
#pragma unroll
                    for (int c = 0; c < KC; c++) accv[c] = BF_WMM(true, 3 * KC * i + 2 * KC + c, fragments(xq, act, 8 * c));
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float st[KC];
#pragma unroll
                    for (int c = 0; c < KC; c++) st[c] = AHEAD ? sa_tok[c][r] : __shfl(sa[c], ch(r, g));
                    vf[r] = chunk_sum<KC, BIASED>(accv, r, st) * swv + bv;
                }
                if (TAPS && a.taps.acc_qkv)
#pragma unroll
                    for (int c = 0; c < KC; c++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            int* row = a.taps.acc_qkv + ((bl * KC + c) * T + t) * 3 * D;
                            row[32 * h + ch(r, g)] = tapbits<BIASED>(accq[c], r);
                            row[D + 32 * h + ch(r, g)] = tapbits<BIASED>(acck[c], r);
                            a.taps.acc_qkv[((bl * KC + c) * T + ch(r, g)) * 3 * D + 2 * D + 32 * h + t] = tapbits<BIASED>(accv[c], r);
                        }
            }
            BF_PHASE(PH_QKV);
            // scores, transposed: lane = query token, register r = key ch(r, g)
            v16f sc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 16; r++) sc = BF_F32MMA(kf[r], qf[r], sc);
            if (AHEAD && i + 1 < TWW) {
#pragma unroll
                for (int c = 0; c < KC; c++) accq[c] = BF_WMM(false, 3 * KC * (i + 1) + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int c = 0; c < KC; c++) acck[c] = BF_WMM(false, 3 * KC * (i + 1) + KC + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int c = 0; c < KC; c++) accv[c] = BF_WMM(true, 3 * KC * (i + 1) + 2 * KC + c, fragments(xq, act, 8 * c));
            }
            float p[16];
            float mx = -__builtin_inff();
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float s = sc[r] * 0.17677669529663687f;
                s = ((alive >> ch(r, g)) & 1u) ? s : -__builtin_inff();
                p[r] = s;
                mx = __builtin_fmaxf(mx, s);
            }
            mx = __builtin_fmaxf(mx, partner(mx, g));
            float lsum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                p[r] = exp_neg(p[r] - mx);
                lsum = lsum + p[r];
            }
            const float rl = 1.0f / (lsum + partner(lsum, g));
            v16f oa = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 16; r++) oa = BF_F32MMA(vf[r], p[r] * rl, oa);
#pragma unroll
            for (int r = 0; r < 16; r++) o[i][r] = oa[r];
            BF_PHASE(PH_ATTN);
        }

        // ---- output projection + residual (this wave's output tiles) -----------------------------------
        {
            v4i oq[NT];
            float so[KC];
            quant_exchange(o, so, oq, TAPS ? a.taps.qa_out : nullptr, bl);
            constexpr int K0 = 3 * KC * TWW;
            acc_t acc2[2][KC];
#pragma unroll
            for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, K0 + c, fragments(oq, act, 8 * c));
#pragma unroll
            for (int i = 0; i < TWW; i++) {
                if (AHEAD && i + 1 < TWW)
#pragma unroll
                    for (int c = 0; c < KC; c++) acc2[(i + 1) & 1][c] = BF_WMM(false, K0 + KC * (i + 1) + c, fragments(oq, act, 8 * c));
                v4f bo[4];
                load_tile16(pA + C::A_BOUT + 32 * (t0 + i), g, bo);
                const float sw = pA[C::A_SW + 3 * TW + t0 + i];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        x[i][4 * j + k] = x[i][4 * j + k] + (chunk_sum<KC, BIASED>(acc2[AHEAD ? i & 1 : 0], 4 * j + k, so) * sw + bo[j][k]);
                pin16(x[i]);
                if (TAPS && a.taps.acc_out)
#pragma unroll
                    for (int c = 0; c < KC; c++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            a.taps.acc_out[((bl * KC + c) * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = tapbits<BIASED>(acc2[AHEAD ? i & 1 : 0][c], r);
                if (!AHEAD && i + 1 < TWW)
#pragma unroll
                    for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, K0 + KC * (i + 1) + c, fragments(oq, act, 8 * c));
            }
        }
        BF_PHASE(PH_OUT);
        // the attention-phase parameters are dead for this wave: fetch the next layer's (a shared
        // copy: after the next barriers, which the quarter's other wave reaches when it is done too)
        if constexpr (!SHARED_PAR) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)lnext * C::PW_FLOATS, pA, C::A_FLOATS, lane);
        }

        // ---- feed-forward --------------------------------------------------------------------------------
        {
            float y[TWW][16];
            layernorm(x, pB + C::B_LN2G + 32 * t0, pB + C::B_LN2B + 32 * t0, y);
            quant_exchange(y, sa, xq, TAPS ? a.taps.qa_ff1 : nullptr, bl);
        }
        if (SHARED_PAR && par_owner) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)lnext * C::PW_FLOATS, pA, C::A_FLOATS, lane);
        }
        BF_PHASE(PH_LN2);
        constexpr int KF = 3 * KC * TWW + KC * TWW;   // the wave's first feed-forward block of the layer
        if constexpr (FULLHID) {
            // First matmul of every step, each step's two 256-wide chunks quantised as soon as the
            // step is complete (a chunk spans a pair of quarters: waves 0,1 the step's first chunk,
            // 2,3 its second); the whole quantised hidden row stays in LDS.  int8: unsigned, bytes
            // stored as q - 128 for the signed MFMA; e4m3: the ordinary signed quantiser.
            float sh[KCF];
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                const int k1 = KF + st * HT * KC;
                float hf[HT][16];
                float am = 0.0f;
                acc_t acc2[2][KC];
#pragma unroll
                for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, k1 + c, fragments(xq, act, 8 * c));
#pragma unroll
                for (int i = 0; i < HT; i++) {
                    if (AH_FFN && i + 1 < HT)
#pragma unroll
                        for (int c = 0; c < KC; c++) acc2[(i + 1) & 1][c] = BF_WMM(false, k1 + KC * (i + 1) + c, fragments(xq, act, 8 * c));
                    v4f b1[4];
                    load_tile16(pBt + C::B_BFF1 + 128 * st + 32 * (h0 + i), g, b1);
                    const float sw = pB[C::B_SW + 4 * st + h0 + i];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            // int8: the ReLU is the saturation of the unsigned quantiser below, and the
                            // running maximum starts at 0, so negative values need no clamp here
                            float v = chunk_sum<KC, BIASED>(acc2[AH_FFN ? i & 1 : 0], 4 * j + k, sa) * sw + b1[j][k];
                            if constexpr (FP8) v = __builtin_fmaxf(v, 0.0f);
                            hf[i][4 * j + k] = v;
                            am = __builtin_fmaxf(am, v);
                        }
                    pin16(hf[i]);
                    if (TAPS && a.taps.acc_ff1)
#pragma unroll
                        for (int c = 0; c < KC; c++)
#pragma unroll
                            for (int r = 0; r < 16; r++)
                                a.taps.acc_ff1[((bl * KC + c) * T + t) * F + 512 * st + 128 * q + 32 * (h0 + i) + ch(r, g)] = tapbits<BIASED>(acc2[AH_FFN ? i & 1 : 0][c], r);
                    if (!AH_FFN && i + 1 < HT)
#pragma unroll
                        for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, k1 + KC * (i + 1) + c, fragments(xq, act, 8 * c));
                }
                // the maxima of consecutive steps go through different exchange slots (2, then 0, whose
                // last use was the LayerNorm sum several barriers ago): a fast wave's next maximum
                // must not overwrite what a slow wave still reads
                const int xs = (st & 1) ? 0 : 2 * XS;
                xch[xs + wave * 64 + lane] = am;
                barrier();
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    float m = 0.0f;   // hidden values are >= 0
#pragma unroll
                    for (int u = 0; u < SUB; u++)
                        m = __builtin_fmaxf(m, __builtin_fmaxf(xch[xs + (2 * c + 4 * u) * 64 + lane],
                                                               xch[xs + (2 * c + 1 + 4 * u) * 64 + lane]));
                    m = __builtin_fmaxf(m, partner(m, g));
                    sh[2 * st + c] = m > 0.0f ? (FP8 ? m * 0.125f : div255(m)) : 1.0f;
                }
                const float s8 = q < 2 ? sh[2 * st] : sh[2 * st + 1];
                const float inv = 1.0f / s8;
#pragma unroll
                for (int i = 0; i < HT; i++) {
                    v4i w;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        unsigned u;
                        if constexpr (FP8) u = quant4<true>(hf[i][4 * j], hf[i][4 * j + 1], hf[i][4 * j + 2], hf[i][4 * j + 3], s8, inv);
                        else u = quant4_relu_u8(hf[i][4 * j], hf[i][4 * j + 1], hf[i][4 * j + 2], hf[i][4 * j + 3], s8, inv);
                        if (TAPS && a.taps.qa_ff2)
                            *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl * T + t) * F + 512 * st + 128 * q + 32 * (h0 + i) + 8 * j + 4 * g) = u;
                        w[j] = (int)(FP8 ? u : (u ^ 0x80808080u));
                    }
                    *reinterpret_cast<v4i*>(hid + (16 * st + 4 * q + h0 + i) * FRAG + lane * 16) = w;
                }
            }
            barrier();   // the whole hidden row is in LDS
            BF_PHASE(PH_FF1);
            // Second matmul, tile by tile: the KCF k-chunks of one output tile in turn, so only one
            // tile's sums over the chunks (float64 for int8, fp32 for e4m3) are alive.  int8: the
            // accumulator starts at 128 * sum(w), the offset of the unsigned bytes stored as q - 128.
            constexpr int K2 = KF + STEPS * HT * KC, N2 = TWW * KCF;
            auto wsum_start = [&](int idx) -> acc_t {
                acc_t r = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                if constexpr (!FP8) {
                    v4i w0[4];
                    load_tile16i(pBt + C::B_WSUM + (idx % KCF) * CW + 32 * (t0 + idx / KCF), g, w0);
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int k = 0; k < 4; k++) r[4 * j + k] = w0[j][k];
                }
                return r;
            };
            auto product = [&](int idx) -> acc_t {
                const int cc = idx % KCF;
                v4i hqc[8];
                if constexpr (!ACTL)
#pragma unroll
                    for (int s = 0; s < 8; s++) hqc[s] = *reinterpret_cast<const v4i*>(hid + (8 * cc + s) * FRAG + lane * 16);
                return BF_WMM_FROM(false, K2 + idx, (FragSrc{&hqc[0], hid + 8 * cc * FRAG + lane * 16}), wsum_start(idx));
            };
            acc_t accp[2];
            accp[0] = product(0);
            double o64[16];
            float o32[16];
#pragma unroll
            for (int idx = 0; idx < N2; idx++) {
                const int i = idx / KCF, cc = idx % KCF;
                if (AH_FFN && idx + 1 < N2) accp[(idx + 1) & 1] = product(idx + 1);
                const acc_t acc = accp[AH_FFN ? idx & 1 : 0];
                if constexpr (FP8) {
                    // descale each 256-deep tile with its own scales, fp32 sum over the tiles
                    const float sw = pB[C::B_SW + 16 + (t0 + i) * KCF + cc];
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const float part = (accf(acc, r) * sh[cc]) * sw;
                        o32[r] = cc == 0 ? part : o32[r] + part;
                        if (TAPS && a.taps.acc_ff2)
                            a.taps.acc_ff2[((bl * KCF + cc) * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = accbits(acc, r);
                    }
                    pin16(o32);
                } else {
                    const double sc = (double)sh[cc];
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int full = accbits(acc, r);
                        o64[r] = cc == 0 ? (double)full * sc : __builtin_fma((double)full, sc, o64[r]);
                        if (TAPS && a.taps.acc_ff2)
                            a.taps.acc_ff2[((bl * KCF + cc) * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = full;
                    }
#pragma unroll
                    for (int r = 0; r < 16; r++) pin(o64[r]);
                }
                if (cc == KCF - 1) {
                    v4f b2[4];
                    load_tile16(pB + C::B_BFF2 + 32 * (t0 + i), g, b2);
                    const float sw = pB[C::B_SW + 16 + t0 + i];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            float upd;
                            if constexpr (FP8) upd = o32[4 * j + k] + b2[j][k];
                            else upd = (float)o64[4 * j + k] * sw + b2[j][k];
                            x[i][4 * j + k] = x[i][4 * j + k] + upd;
                        }
                    pin16(x[i]);
                }
                if (!AH_FFN && idx + 1 < N2) accp[0] = product(idx + 1);
            }
            BF_PHASE(PH_FF2);
        } else {
            double o64[TWW][16];   // int8: float64 sums over the k-chunks
            float o32[TWW][16];    // e4m3: fp32 sums over the k-tiles
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                constexpr int SBLK = HT * KC + 2 * TWW;   // the wave's blocks of one step
                const int k1 = KF + st * SBLK;            // first matmul: HT hidden tiles of this wave (of the 16 of a step)
                float sh[2];                              // scales of the step's two chunks
                {
                    float hf[HT][16];
                    float am = 0.0f;
                    acc_t acc2[2][KC];
#pragma unroll
                    for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, k1 + c, fragments(xq, act, 8 * c));
#pragma unroll
                    for (int i = 0; i < HT; i++) {
                        if (AHEAD && i + 1 < HT)
#pragma unroll
                            for (int c = 0; c < KC; c++) acc2[(i + 1) & 1][c] = BF_WMM(false, k1 + KC * (i + 1) + c, fragments(xq, act, 8 * c));
                        v4f b1[4];
                        load_tile16(pBt + C::B_BFF1 + 128 * st + 32 * (h0 + i), g, b1);
                        const float sw = pB[C::B_SW + 4 * st + h0 + i];
#pragma unroll
                        for (int j = 0; j < 4; j++)
#pragma unroll
                            for (int k = 0; k < 4; k++) {
                                // int8: the ReLU is the saturation of the unsigned quantiser below, and the
                                // running maximum starts at 0, so negative values need no clamp here
                                float v = chunk_sum<KC, BIASED>(acc2[AHEAD ? i & 1 : 0], 4 * j + k, sa) * sw + b1[j][k];
                                if constexpr (FP8) v = __builtin_fmaxf(v, 0.0f);
                                hf[i][4 * j + k] = v;
                                am = __builtin_fmaxf(am, v);
                            }
                        pin16(hf[i]);
                        if (TAPS && a.taps.acc_ff1)
#pragma unroll
                            for (int c = 0; c < KC; c++)
#pragma unroll
                                for (int r = 0; r < 16; r++)
                                    a.taps.acc_ff1[((bl * KC + c) * T + t) * F + 512 * st + 128 * q + 32 * (h0 + i) + ch(r, g)] = tapbits<BIASED>(acc2[AHEAD ? i & 1 : 0][c], r);
                        if (!AHEAD && i + 1 < HT)
#pragma unroll
                            for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, k1 + KC * (i + 1) + c, fragments(xq, act, 8 * c));
                    }
                    // quantiser over the 256-wide chunk this wave shares with its neighbour (waves 0,1: first
                    // chunk of the step; 2,3: second).  int8: unsigned, bytes stored as q - 128 for the signed
                    // MFMA; e4m3: the ordinary signed quantiser (the values are non-negative)
                    xch[2 * XS + wave * 64 + lane] = am;
                    barrier();
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        float m = 0.0f;   // hidden values are >= 0
#pragma unroll
                        for (int u = 0; u < SUB; u++)
                            m = __builtin_fmaxf(m, __builtin_fmaxf(xch[2 * XS + (2 * c + 4 * u) * 64 + lane],
                                                                   xch[2 * XS + (2 * c + 1 + 4 * u) * 64 + lane]));
                        m = __builtin_fmaxf(m, partner(m, g));
                        sh[c] = m > 0.0f ? (FP8 ? m * 0.125f : div255(m)) : 1.0f;
                    }
                    const float s8 = q < 2 ? sh[0] : sh[1];
                    const float inv = 1.0f / s8;
#pragma unroll
                    for (int i = 0; i < HT; i++) {
                        v4i w;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            unsigned u;
                            if constexpr (FP8) u = quant4<true>(hf[i][4 * j], hf[i][4 * j + 1], hf[i][4 * j + 2], hf[i][4 * j + 3], s8, inv);
                            else u = quant4_relu_u8(hf[i][4 * j], hf[i][4 * j + 1], hf[i][4 * j + 2], hf[i][4 * j + 3], s8, inv);
                            if (TAPS && a.taps.qa_ff2)
                                *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl * T + t) * F + 512 * st + 128 * q + 32 * (h0 + i) + 8 * j + 4 * g) = u;
                            w[j] = (int)(FP8 ? u : (u ^ 0x80808080u));
                        }
                        *reinterpret_cast<v4i*>(hid + (4 * q + h0 + i) * FRAG + lane * 16) = w;
                    }
                }
                barrier();
                BF_PHASE(PH_FF1);
                // second matmul, chunk-major: one chunk of the hidden row (eight fragments) serves this
                // wave's TW output tiles; the float64 sums over the chunks stay in chunk order
                const int k2 = k1 + HT * KC;
                acc_t acc2[2];
                v4i hqc[8];
                if constexpr (!ACTL)
#pragma unroll
                    for (int s = 0; s < 8; s++) hqc[s] = *reinterpret_cast<const v4i*>(hid + s * FRAG + lane * 16);
                // int8, one product at a time: the accumulator starts at 128 * sum(w) (the offset of the
                // unsigned operand bytes stored as q - 128), which saves adding it afterwards
                constexpr bool WFOLD = !AHEAD && !FP8;
                auto wsum_start = [&](int idx) -> acc_t {
                    acc_t r = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    if constexpr (WFOLD) {
                        v4i w0[4];
                        load_tile16i(pBt + C::B_WSUM + (2 * st + idx / TWW) * CW + 32 * (t0 + idx % TWW), g, w0);
#pragma unroll
                        for (int j = 0; j < 4; j++)
#pragma unroll
                            for (int k = 0; k < 4; k++) r[4 * j + k] = w0[j][k];
                    }
                    return r;
                };
                acc2[0] = BF_WMM_FROM(false, k2, fragments(hqc, hid, 0), wsum_start(0));
#pragma unroll
                for (int idx = 0; idx < 2 * TWW; idx++) {
                    const int c = idx / TWW, i = idx % TWW;
                    v4i ws[4] = {};
                    if (!FP8 && !WFOLD) load_tile16i(pBt + C::B_WSUM + (2 * st + c) * CW + 32 * (t0 + i), g, ws);
                    if (AHEAD && idx + 1 < 2 * TWW) {
                        if ((idx + 1) % TWW == 0)
#pragma unroll
                            for (int s = 0; s < 8; s++)
                                hqc[s] = *reinterpret_cast<const v4i*>(hid + (8 * (c + 1) + s) * FRAG + lane * 16);
                        acc2[(idx + 1) & 1] = BF_WMM(false, k2 + idx + 1, fragments(hqc, hid, 0));
                    }
                    if (!AHEAD && idx > 0) {
                        if (!ACTL && idx % TWW == 0)   // the next chunk of the hidden row
#pragma unroll
                            for (int s = 0; s < 8; s++)
                                hqc[s] = *reinterpret_cast<const v4i*>(hid + (8 * c + s) * FRAG + lane * 16);
                        acc2[0] = BF_WMM_FROM(false, k2 + idx, (FragSrc{&hqc[0], hid + 8 * c * FRAG + lane * 16}), wsum_start(idx));
                    }
                    const acc_t acc = acc2[AHEAD ? idx & 1 : 0];
                    if constexpr (FP8) {
                        // descale each 256-deep tile with its own scales, fp32 sum over the tiles
                        const float sw = pB[C::B_SW + 16 + (t0 + i) * KCF + 2 * st + c];
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const float part = (accf(acc, r) * sh[c]) * sw;
                            o32[i][r] = (st == 0 && c == 0) ? part : o32[i][r] + part;
                            if (TAPS && a.taps.acc_ff2)
                                a.taps.acc_ff2[((bl * KCF + 2 * st + c) * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = accbits(acc, r);
                        }
                        pin16(o32[i]);
                    } else {
                        const double sc = (double)sh[c];
#pragma unroll
                        for (int j = 0; j < 4; j++)
#pragma unroll
                            for (int k = 0; k < 4; k++) {
                                const int full = WFOLD ? accbits(acc, 4 * j + k) : accbits(acc, 4 * j + k) + ws[j][k];
                                o64[i][4 * j + k] = (st == 0 && c == 0) ? (double)full * sc
                                                                        : __builtin_fma((double)full, sc, o64[i][4 * j + k]);
                                if (TAPS && a.taps.acc_ff2)
                                    a.taps.acc_ff2[((bl * KCF + 2 * st + c) * T + t) * D + 32 * (TW * q + t0 + i) + 8 * j + 4 * g + k] = full;
                            }
#pragma unroll
                        for (int r = 0; r < 16; r++) pin(o64[i][r]);
                    }
                }
                BF_PHASE(PH_FF2);
            }
#pragma unroll
            for (int i = 0; i < TWW; i++) {
                v4f b2[4];
                load_tile16(pB + C::B_BFF2 + 32 * (t0 + i), g, b2);
                const float sw = pB[C::B_SW + 16 + t0 + i];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        float upd;
                        if constexpr (FP8) upd = o32[i][4 * j + k] + b2[j][k];
                        else upd = (float)o64[i][4 * j + k] * sw + b2[j][k];
                        x[i][4 * j + k] = x[i][4 * j + k] + upd;
                    }
            }
        }
        if constexpr (!SHARED_PAR) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)lnext * C::PW_FLOATS + C::A_FLOATS, pB, B_COPY, lane);
        }
        BF_PHASE(PH_FF2);
#undef BF_WMM
#undef BF_WMM_FROM
        if (TAPS && a.taps.resid)
#pragma unroll
            for (int i = 0; i < TWW; i++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    a.taps.resid[(bl * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = x[i][r];
    }
    if (TAPS && a.taps.resid_last)
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.resid_last[((size_t)b * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = x[i][r];
    if (enc_only) return;   // the same for every wave of the launch

    // ---- final norm and heads --------------------------------------------------------------------------
    // The first head block is in the fragment registers unless a layer range that stops early left
    // the blocks of the next layer there: then restart the stream at the head blocks.
    const int hseq0 = (a.n_layers - a.l0) * BPW;
    wait_vm<0>();   // also: no parameter copy is still landing where the normalised stream goes
    if (OCTO || a.l1 != a.n_layers || (TWIN && nl_run == 0)) {
        if constexpr (TWIN) {
#pragma unroll
            for (int j = 0; j < NSETS - 1; j++) load_half(2 * hseq0 + j, j);
        } else {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < SLOTS; j++) issue_block(hseq0 + j, j);
            wait_vm<0>();
            read_slot(0);
        }
    }
    float hn[TWW][16];
    layernorm(x, gp + C::G_NFG + CW * q + 32 * t0, gp + C::G_NFB + CW * q + 32 * t0, hn);
    if (TAPS && a.taps.normed)
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.normed[((size_t)b * T + t) * D + 32 * (TW * q + t0 + i) + ch(r, g)] = hn[i][r];
    // publish as B-operand fragments (n, j): lane holds the four floats of register quad j
    float* const hnb = reinterpret_cast<float*>(hid);
#pragma unroll
    for (int i = 0; i < TWW; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v4f v = {hn[i][4 * j], hn[i][4 * j + 1], hn[i][4 * j + 2], hn[i][4 * j + 3]};
            *reinterpret_cast<v4f*>(hnb + (((TW * q + t0 + i) * 4 + j) * 64 + lane) * 4) = v;
        }
    barrier();
    // The first wave of quarter m multiplies head tile m (rows 32m..32m+31 of [policy; promo;
    // value; 0]) over the whole width, one fused-multiply-add chain in (tile, quad, element) order;
    // quarter 3's tile is zero.  With eight waves the second wave of a quarter has nothing to
    // do here but meet the barrier of the argmax exchange.
    const bool heads_here = !OCTO || sub == 0;
    v16f head = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if (!heads_here) {
    } else if constexpr (TWIN) {
#pragma unroll
        for (int hi = 0; hi < 2 * HB; hi++) {          // half-block = the four fragments (n = hi, q = 0..3)
            // the stream is padded by one block: two half-blocks past the last head block exist
            if (hi + NSETS - 1 < 2 * HB + 2) load_half(2 * hseq0 + hi + NSETS - 1, (hi + NSETS - 1) % NSETS);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const v4f w = __builtin_bit_cast(v4f, frt[hi % NSETS][s]);
                const v4f hv = *reinterpret_cast<const v4f*>(hnb + ((hi * 4 + s) * 64 + lane) * 4);
#pragma unroll
                for (int k = 0; k < 4; k++) head = __builtin_amdgcn_mfma_f32_32x32x2f32(w[k], hv[k], head, 0, 0, 0);
            }
        }
    } else {
#pragma unroll
        for (int hb = 0; hb < HB; hb++) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (hb + SLOTS < HB) issue_block(hseq0 + hb + SLOTS, hb % SLOTS);
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const v4f w = __builtin_bit_cast(v4f, fr[s]);
                const v4f hv = *reinterpret_cast<const v4f*>(hnb + ((hb * 8 + s) * 64 + lane) * 4);
#pragma unroll
                for (int k = 0; k < 4; k++) head = __builtin_amdgcn_mfma_f32_32x32x2f32(w[k], hv[k], head, 0, 0, 0);
            }
            if (hb + 1 < HB) {
                wait_vm<0>();
                read_slot((hb + 1) % SLOTS);
            }
        }
    }

    BF_PHASE(PH_HEADS);
    // raw value logits (registers 0..2 of a lane of head tile 2's upper half) to the value in [-1, 1]
    auto value_of = [&](const v16f& hd) -> float {
        if (a.n_value == 1) return tanh_dev(hd[0]);
        const float r0 = hd[0], r1 = hd[1], r2 = hd[2];   // classes loss, draw, win
        const float mx = __builtin_fmaxf(__builtin_fmaxf(r0, r1), r2);
        const float e0 = exp_neg(r0 - mx), e1 = exp_neg(r1 - mx), e2 = exp_neg(r2 - mx);
        return (e2 - e0) / ((e0 + e1) + e2);
    };
    // value (king head): king token of the side to move, lane half 1 of head tile 2 holds rows 68..70
    if (heads_here && q == 2) {
        const int king = ctrl < 0 ? 31 : 15;
        if (a.vmode == 0 && lane == 32 + king) a.value[b] = value_of(head);
        if (g == 0) {   // promo: rows 64..67 are registers 0..3 of lane half 0
            if (a.out_fp32) {
                const v4f v = {head[0], head[1], head[2], head[3]};
                *reinterpret_cast<v4f*>((float*)a.promo + ((size_t)b * T + t) * 4) = v;
            } else {
                const v4h v = {(_Float16)head[0], (_Float16)head[1], (_Float16)head[2], (_Float16)head[3]};
                *reinterpret_cast<v4h*>((_Float16*)a.promo + ((size_t)b * T + t) * 4) = v;
            }
        }
    }
    // policy (waves 0 and 1: squares 0..31 and 32..63), optional legal-move AND and argmax
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    if (heads_here && q < 2) {
        unsigned long long mw = ~0ull;
        if (a.mask) mw = a.mask[(size_t)b * T + t];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int sq = 32 * q + 8 * j + 4 * g + k;
                const bool legal = (mw >> sq) & 1ull;
                v[k] = legal ? head[4 * j + k] : -__builtin_inff();
                // squares are visited in increasing order within a lane, so '>' keeps the lowest
                if (legal && (bi == 0x7fffffff || v[k] > bv)) { bv = v[k]; bi = t * 64 + sq; }
            }
            const size_t at = ((size_t)b * T + t) * 64 + 32 * q + 8 * j + 4 * g;
            if (a.out_fp32) {
                const v4f vv = {v[0], v[1], v[2], v[3]};
                *reinterpret_cast<v4f*>((float*)a.policy + at) = vv;
            } else {
                const v4h vv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                *reinterpret_cast<v4h*>((_Float16*)a.policy + at) = vv;
            }
        }
    }
    if (a.mask && a.best) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            const float ov = __shfl_xor(bv, d);
            const int oi = __shfl_xor(bi, d);
            const bool take = (oi != 0x7fffffff) && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
            bv = take ? ov : bv;
            bi = take ? oi : bi;
        }
        // the two policy waves' winners meet in the exchange area (its last use was long ago)
        if (heads_here && lane == 0) {
            xch[q * 2] = bv;
            xch[q * 2 + 1] = __int_as_float(bi);
        }
        barrier();
        if (wave == 0 && lane == 0) {
            const float ov = xch[2];
            const int oi = __float_as_int(xch[3]);
            const bool take = (oi != 0x7fffffff) && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
            bi = take ? oi : bi;
            a.best[b] = bi == 0x7fffffff ? -1 : bi;
        }
    }
    // ---- pooled value heads (reference brokefish/nn/model.py:576-617) --------------------------------
    // The value row is the mean over the live tokens of the normalised stream ("pooled", mode 1) or
    // the final LayerNorm of the mean of the residual stream ("prenorm", mode 2); it goes through
    // the value rows of head tile 2 like a token, and the result is in White's frame, so it is
    // negated when Black is to move.  The token sum is a butterfly over the 32 lanes of a half
    // (distances 16, 8, 4, 2, 1), which leaves the pooled row in every lane in a token row's layout.
    if (a.vmode != 0) {
        const bool live = (alive >> t) & 1u;
        const float cdiv = (float)(__builtin_popcount(alive) > 0 ? __builtin_popcount(alive) : 1);
        float pv[TWW][16], hv[TWW][16];
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float v = live ? (a.vmode == 1 ? hn[i][r] : x[i][r]) : 0.0f;
#pragma unroll
                for (int d = 16; d >= 1; d >>= 1) v = v + __shfl_xor(v, d);
                pv[i][r] = v / cdiv;
            }
        if (a.vmode == 2) {
            layernorm(pv, gp + C::G_NFG + CW * q + 32 * t0, gp + C::G_NFB + CW * q + 32 * t0, hv);
        } else {
#pragma unroll
            for (int i = 0; i < TWW; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) hv[i][r] = pv[i][r];
        }
        barrier();   // every wave has finished reading the normalised stream
#pragma unroll
        for (int i = 0; i < TWW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = {hv[i][4 * j], hv[i][4 * j + 1], hv[i][4 * j + 2], hv[i][4 * j + 3]};
                *reinterpret_cast<v4f*>(hnb + (((TW * q + t0 + i) * 4 + j) * 64 + lane) * 4) = v;
            }
        barrier();
        if (heads_here && q == 2) {
            // head tile 2 once more, against the pooled row (every token column holds the same row);
            // its blocks are read straight from the stream, in the same order as above
            v16f hd = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            for (int f = 0; f < 8 * HB; f++) {
                const v4f w = *reinterpret_cast<const v4f*>(wsrc + (size_t)hseq0 * BLOCK + (size_t)f * FRAG);
                const v4f hvv = *reinterpret_cast<const v4f*>(hnb + (f * 64 + lane) * 4);
#pragma unroll
                for (int k = 0; k < 4; k++) hd = __builtin_amdgcn_mfma_f32_32x32x2f32(w[k], hvv[k], hd, 0, 0, 0);
            }
            if (lane == 32) {
                const float v = value_of(hd);
                a.value[b] = ctrl > 0 ? v : -v;
            }
        }
    }
    if constexpr (PROF) {
        BF_PHASE(PH_STORE);
        ph[PH_SYNC] = t_sync;
        ph[PH_TOTAL] = __builtin_readcyclecounter() - t_begin;
        if (lane == 0 && a.profile)
#pragma unroll
            for (int i = 0; i < N_PHASES; i++) atomicAdd(&a.profile[i], ph[i]);
    }
#undef BF_PHASE
}

template <int DM, bool TAPS, bool TWIN, bool FP8 = false, bool OCTO = false, bool PROF = false>
hipError_t launch_board(const KArgs& k, hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be requested once per kernel and device (one bit
    // per device ordinal; a device beyond the mask asks every time)
    static std::atomic<unsigned long long> lds_set{0};
    constexpr int lds_bytes = Cfg<DM, TWIN, OCTO>::LDS_BYTES;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
    if (!(lds_set.load(std::memory_order_relaxed) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&board_kernel<DM, TAPS, TWIN, FP8, OCTO, PROF>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return e;
        lds_set.fetch_or(bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL((board_kernel<DM, TAPS, TWIN, FP8, OCTO, PROF>), dim3(k.n), dim3(OCTO ? 2 * THREADS : THREADS), lds_bytes, stream, k);
    return hipGetLastError();
}

}  // namespace board
}  // namespace bf
