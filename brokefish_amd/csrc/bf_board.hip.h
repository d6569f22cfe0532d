// The evaluator with ONE position per workgroup: the four wavefronts split the model width.
//
// Wavefront w owns a quarter of the channels of the residual stream (tiles TW*w .. TW*w+TW-1,
// which are also its attention heads), a quarter of every matmul's output tiles, and streams
// exactly the weight blocks of those tiles -- privately, so weights need no cross-wave
// synchronisation.  Quantised activations are exchanged through LDS as ready-made MFMA
// B-operand fragments; row statistics (LayerNorm sums, quantiser maxima) are exchanged as
// per-lane partials and combined in wave order, which is the group order of the arithmetic
// contract in bf_args.h -- so for the 256-wide network this kernel returns bit for bit what the
// one-wavefront-per-position kernel returns.  The feed-forward block runs in steps of 512 hidden
// channels: each wave computes four hidden tiles per step, so a 256-wide quantiser chunk spans a
// pair of waves and its maximum is exchanged; the float64 sums over the chunks stay in order.
//
// Two forms, selected by TWIN, with identical results:
//   TWIN = false  one workgroup per compute unit, 512 registers per wave.  Weight blocks stream
//                 through a private LDS ring per wave (direct-to-LDS loads, SLOTS blocks deep),
//                 attention is software-pipelined across heads.  Lowest latency per position
//                 (launches of up to one position per compute unit) and the only form the
//                 512-wide network fits.
//   TWIN = true   two workgroups per compute unit: at most 80 KiB of LDS and 256 registers per
//                 wave, so every SIMD holds two wavefronts of different positions and one's
//                 waits (LDS round trips, barriers, MFMA results) are covered by the other's
//                 work.  Weight fragments go from L2 straight to registers (half a block = four
//                 fragments at a time, prefetched through a rotation of register sets).
//                 Highest throughput.
//
// LDS map (bytes): [ring: 4 waves x SLOTS x 8 KiB, absent in the TWIN form] [xch: 3 KiB]
// [hid: 16 KiB] [act: NT KiB] [par: 4 waves x PW floats].  During the heads the normalised stream
// (NT*4 KiB, fp32) overlays hid/act/par.
#pragma once

#include "bf_device.hip.h"

// TWIN form: workgroups per compute unit, and register sets of the weight prefetch (one set =
// half a block; SETS - 1 half-blocks are in flight).  Measured on MI355X at batch 4096: three
// workgroups per unit spill too much (1.42 M evals/s against 2.10 M), four sets beat three by 2 %.
#ifndef BF_TWIN_SETS
#define BF_TWIN_SETS 4
#endif
#ifndef BF_TWIN_OCC
#define BF_TWIN_OCC 2
#endif

namespace bf {
namespace board {

extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

template <int DM, bool TWIN>
struct Cfg : Layout<DM> {
    typedef Layout<DM> L;
    static constexpr int RING_BYTES = TWIN ? 0 : 4 * L::SLOTS * BLOCK;
    static constexpr int XCH_OFF = RING_BYTES;
    static constexpr int HID_OFF = XCH_OFF + 3 * FRAG;
    static constexpr int ACT_OFF = HID_OFF + 16 * FRAG;
    static constexpr int PAR_OFF = ACT_OFF + L::NT * FRAG;
    static constexpr int LDS_BYTES = PAR_OFF + 4 * L::PW_FLOATS * 4;
    static_assert(LDS_BYTES <= (TWIN ? 160 / BF_TWIN_OCC : 160) * 1024, "LDS budget: one or two workgroups per compute unit");
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
// is the same number)
template <int KC, typename ACC>
__device__ __forceinline__ float chunk_sum(const ACC (&acc)[KC], int i, const float (&sa)[KC]) {
    if constexpr (KC == 1) {
        return accf(acc[0], i) * sa[0];
    } else {
        double o = (double)acc[0][i] * (double)sa[0];
#pragma unroll
        for (int c = 1; c < KC; c++) o = __builtin_fma((double)acc[c][i], (double)sa[c], o);
        return (float)o;
    }
}

template <int DM, bool TAPS, bool TWIN, bool FP8>
__global__ __launch_bounds__(THREADS, TWIN ? BF_TWIN_OCC : 1) void board_kernel(const KArgs a) {
    typedef Cfg<DM, TWIN> C;
    typedef typename Acc<FP8>::type acc_t;
    static_assert(!FP8 || DM == 256, "e4m3: one k-chunk per matmul of the width (fp32 sums over the chunks of ffn2 only)");
    constexpr int D = C::D, F = C::F, NT = C::NT, TW = C::TW, CW = C::CW, KC = C::KC, KCF = C::KCF;
    constexpr int STEPS = C::STEPS, BPW = C::BPW, HB = C::HB, SLOTS = C::SLOTS, WPC = 4 / KC;
    constexpr int HALF = BLOCK / 2;   // four fragments: the unit of the register prefetch (TWIN)
    constexpr int NSETS = BF_TWIN_SETS;   // register sets of the prefetch: NSETS - 1 half-blocks in flight
    constexpr int VM_AHEAD = TAPS ? 0 : (SLOTS - 1) * 8;   // ring loads that may stay in flight at a ring wait
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = lane & 31, g = lane >> 5;
    const int b = blockIdx.x;
    if (a.active && !a.active[b]) return;   // a skipped position: the whole workgroup leaves before any barrier
    const int nl_run = a.l1 - a.l0;

    uint8_t* const myring = lds + wave * (SLOTS * BLOCK);   // !TWIN
    float* const xch = reinterpret_cast<float*>(lds + C::XCH_OFF);
    uint8_t* const hid = lds + C::HID_OFF;
    uint8_t* const act = lds + C::ACT_OFF;
    float* const pA = reinterpret_cast<float*>(lds + C::PAR_OFF) + wave * C::PW_FLOATS;
    float* const pB = pA + C::A_FLOATS;
    // this wave's weight stream, from the first layer that runs; block `seq` in consumption order
    const uint8_t* const wsrc =
        a.wstream + ((size_t)wave * ((size_t)a.n_layers * BPW + HB + 1) + (size_t)a.l0 * BPW) * BLOCK + lane * 16;
    const float* const wpar = a.fparams + (size_t)wave * a.n_layers * C::PW_FLOATS;   // this wave's [layer][PW]
    const float* const gp = a.fparams + (size_t)4 * a.n_layers * C::PW_FLOATS;       // tables, final norm

    // TWIN: half-block `hseq` of this wave's stream (consumption order) into register set `set`
    v4i frt[NSETS][4];
    auto load_half = [&](int hseq, int set) {
        const uint8_t* src = wsrc + (size_t)hseq * HALF;
#pragma unroll
        for (int s = 0; s < 4; s++) frt[set][s] = *reinterpret_cast<const v4i*>(src + s * FRAG);
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
    // sum of a per-lane value over the four waves, in wave order
    auto xsum = [&](float v, int slot) -> float {
        xch[slot * 256 + wave * 64 + lane] = v;
        lds_barrier();
        const float* p = xch + slot * 256 + lane;
        return ((p[0] + p[64]) + p[128]) + p[192];
    };
    // LayerNorm of this wave's channels; gamma / beta point at this wave's slice
    auto layernorm = [&](const float (&x)[TW][16], const float* gamma, const float* beta, float (&y)[TW][16]) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) s = s + x[i][r];
        s = xsum(s, 0);
        const float mean = (s + partner(s, g)) * (1.0f / D);
        float v = 0.0f;
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float d = x[i][r] - mean;
                v = __builtin_fmaf(d, d, v);
            }
        v = xsum(v, 1);
        const float var = (v + partner(v, g)) * (1.0f / D);
        const float rstd = 1.0f / __builtin_sqrtf(var + a.eps);
#pragma unroll
        for (int i = 0; i < TW; i++)
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
    auto quant_exchange = [&](const float (&y)[TW][16], float (&sa)[KC], v4i (&q)[NT], int8_t* tap, size_t tap_row) {
        float am = 0.0f;
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) am = __builtin_fmaxf(am, __builtin_fabsf(y[i][r]));
        xch[2 * 256 + wave * 64 + lane] = am;
        lds_barrier();
#pragma unroll
        for (int c = 0; c < KC; c++) {
            float m = 0.0f;
#pragma unroll
            for (int w = c * WPC; w < (c + 1) * WPC; w++) m = __builtin_fmaxf(m, xch[2 * 256 + w * 64 + lane]);
            m = __builtin_fmaxf(m, partner(m, g));
            sa[c] = m > 0.0f ? m / (FP8 ? 8.0f : 127.0f) : 1.0f;
        }
        const float so = KC == 1 ? sa[0] : (wave < WPC ? sa[0] : sa[KC - 1]);
        const float inv = 1.0f / so;
#pragma unroll
        for (int i = 0; i < TW; i++) {
            v4i w;
#pragma unroll
            for (int j = 0; j < 4; j++)
                w[j] = (int)quant4<FP8>(y[i][4 * j], y[i][4 * j + 1], y[i][4 * j + 2], y[i][4 * j + 3], so, inv);
            *reinterpret_cast<v4i*>(act + (TW * wave + i) * FRAG + lane * 16) = w;
            if (TAPS && tap)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(tap + (tap_row * T + t) * D + 32 * (TW * wave + i) + 8 * j + 4 * g) = w[j];
        }
        lds_barrier();
#pragma unroll
        for (int n = 0; n < NT; n++) q[n] = *reinterpret_cast<const v4i*>(act + n * FRAG + lane * 16);
    };

    // ---- start the weight stream and the first layer's parameters ------------------------------
    if constexpr (TWIN) {
#pragma unroll
        for (int j = 0; j < NSETS - 1; j++) load_half(j, j);
    } else {
#pragma unroll
        for (int j = 0; j < SLOTS; j++) issue_block(j, j);
    }
    if (nl_run > 0) {
        dma(wpar + (size_t)a.l0 * C::PW_FLOATS, pA, C::A_FLOATS, lane);
        dma(wpar + (size_t)a.l0 * C::PW_FLOATS + C::A_FLOATS, pB, C::B_FLOATS, lane);
    }

    // ---- embedding (this wave's channels) --------------------------------------------------------
    float x[TW][16];
    const unsigned word = a.boards[(size_t)b * T + t];
    const int ctrl = a.control[b];
    const unsigned alive = (unsigned)__ballot(((word >> 11) & 1) == 0 && g == 0);
    if (TAPS && a.taps.x_in) {
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = ldg4(a.taps.x_in + ((size_t)b * T + t) * D + 32 * (TW * wave + i) + 8 * j + 4 * g);
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
        const int own = CW * wave + 4 * g;
        const float* e_sq = gp + C::G_SQ + (word & 63) * D + own;
        const float* e_ts = gp + C::G_TS + ts * D + own;
        const float* e_ct = gp + C::G_CT + ct * D + own;
        const float* e_ck = gp + C::G_CLOCK + clock * D + own;
        const float* e_rp = gp + C::G_REP + rp * D + own;
#pragma unroll
        for (int i = 0; i < TW; i++)
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
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.embed[((size_t)b * T + t) * D + 32 * (TW * wave + i) + ch(r, g)] = x[i][r];

    wait_vm<0>();   // the parameters (and the first ring slots) have landed
    if constexpr (!TWIN) read_slot(0);

    for (int l = a.l0; l < a.l1; l++) {
        const int li = l - a.l0;
        const size_t bl = (size_t)b * nl_run + li;   // tap row
        const int lnext = l + 1 < a.l1 ? l + 1 : l;  // after the last layer the same slice is fetched again
        // Multiply by block k of this wave's layer.
        // TWIN: its two halves sit in register sets 2k % NSETS and (2k + 1) % NSETS; a set is refilled
        // with the half-block NSETS positions on once it has been consumed.
        // !TWIN: the block is in `fr`; the ring slot it came from is refilled SLOTS blocks ahead,
        // then block k+1 is read from its slot.
        const int hbase = li * 2 * BPW;
#define BF_WMM(SWAP, k, actp)                                                                        \
    ([&]() -> acc_t {                                                                                \
        const v4i* act_ = (actp);                                                                    \
        acc_t r_ = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};                                 \
        if constexpr (TWIN) {                                                                        \
            load_half(hbase + 2 * (k) + NSETS - 1, (2 * (k) + NSETS - 1) % NSETS);                   \
            _Pragma("unroll") for (int s_ = 0; s_ < 4; s_++)                                         \
                r_ = frag_mma<SWAP>(frt[(2 * (k)) % NSETS][s_], act_[s_], r_);                       \
            load_half(hbase + 2 * (k) + NSETS, (2 * (k) + NSETS) % NSETS);                           \
            _Pragma("unroll") for (int s_ = 0; s_ < 4; s_++)                                         \
                r_ = frag_mma<SWAP>(frt[(2 * (k) + 1) % NSETS][s_], act_[4 + s_], r_);               \
        } else {                                                                                     \
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                       \
            issue_block(li * BPW + (k) + SLOTS, (k) % SLOTS);                                        \
            _Pragma("unroll") for (int s_ = 0; s_ < 8; s_++)                                         \
                r_ = frag_mma<SWAP>(fr[s_], act_[s_], r_);                                           \
            wait_vm<VM_AHEAD>();                                                                     \
            read_slot(((k) + 1) % SLOTS);                                                            \
        }                                                                                            \
        return r_;                                                                                   \
    }())

        // ---- LayerNorm 1, quantise, exchange ----------------------------------------------------------
        v4i xq[NT];
        float sa[KC];
        {
            float y[TW][16];
            layernorm(x, pA + C::A_LN1G, pA + C::A_LN1B, y);
            quant_exchange(y, sa, xq, TAPS ? a.taps.qa_qkv : nullptr, bl);
        }
        float sa_tok[KC][16];   // activation scale of token ch(r, g), for the V tiles whose rows are tokens
#pragma unroll
        for (int c = 0; c < KC; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) sa_tok[c][r] = __shfl(sa[c], ch(r, g));

        // ---- attention over this wave's heads ----------------------------------------------------------
        // !TWIN: software-pipelined -- the three weight GEMMs of head i+1 are issued right after the
        // score MFMAs of head i, so the matrix pipe works through them under head i's softmax.
        float o[TW][16];
        acc_t accq[KC], acck[KC], accv[KC];
#pragma unroll
        for (int i = 0; i < TW; i++) {
            if (TWIN || i == 0) {
#pragma unroll
                for (int c = 0; c < KC; c++) accq[c] = BF_WMM(false, 3 * KC * i + c, &xq[8 * c]);
#pragma unroll
                for (int c = 0; c < KC; c++) acck[c] = BF_WMM(false, 3 * KC * i + KC + c, &xq[8 * c]);
#pragma unroll
                for (int c = 0; c < KC; c++) accv[c] = BF_WMM(true, 3 * KC * i + 2 * KC + c, &xq[8 * c]);
            }
            const int h = TW * wave + i;
            float qf[16], kf[16], vf[16];
            {
                const float swq = pA[C::A_SW + i], swk = pA[C::A_SW + TW + i], swv = pA[C::A_SW + 2 * TW + i];
                const float bv = pA[C::A_BV + 32 * i + t];
                v4f bq[4], bk[4];
                load_tile16(pA + C::A_BQ + 32 * i, g, bq);
                load_tile16(pA + C::A_BK + 32 * i, g, bk);
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        qf[4 * j + k] = chunk_sum<KC>(accq, 4 * j + k, sa) * swq + bq[j][k];
                        kf[4 * j + k] = chunk_sum<KC>(acck, 4 * j + k, sa) * swk + bk[j][k];
                    }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float st[KC];
#pragma unroll
                    for (int c = 0; c < KC; c++) st[c] = sa_tok[c][r];
                    vf[r] = chunk_sum<KC>(accv, r, st) * swv + bv;
                }
                if (TAPS && a.taps.acc_qkv)
#pragma unroll
                    for (int c = 0; c < KC; c++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            int* row = a.taps.acc_qkv + ((bl * KC + c) * T + t) * 3 * D;
                            row[32 * h + ch(r, g)] = accbits(accq[c], r);
                            row[D + 32 * h + ch(r, g)] = accbits(acck[c], r);
                            a.taps.acc_qkv[((bl * KC + c) * T + ch(r, g)) * 3 * D + 2 * D + 32 * h + t] = accbits(accv[c], r);
                        }
            }
            // scores, transposed: lane = query token, register r = key ch(r, g)
            v16f sc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 16; r++) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[r], qf[r], sc, 0, 0, 0);
            if (!TWIN && i + 1 < TW) {
#pragma unroll
                for (int c = 0; c < KC; c++) accq[c] = BF_WMM(false, 3 * KC * (i + 1) + c, &xq[8 * c]);
#pragma unroll
                for (int c = 0; c < KC; c++) acck[c] = BF_WMM(false, 3 * KC * (i + 1) + KC + c, &xq[8 * c]);
#pragma unroll
                for (int c = 0; c < KC; c++) accv[c] = BF_WMM(true, 3 * KC * (i + 1) + 2 * KC + c, &xq[8 * c]);
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
            for (int r = 0; r < 16; r++) oa = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[r], p[r] * rl, oa, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) o[i][r] = oa[r];
        }

        // ---- output projection + residual (this wave's output tiles) -----------------------------------
        {
            v4i oq[NT];
            float so[KC];
            quant_exchange(o, so, oq, TAPS ? a.taps.qa_out : nullptr, bl);
            constexpr int K0 = 3 * KC * TW;
            acc_t acc2[2][KC];
#pragma unroll
            for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, K0 + c, &oq[8 * c]);
#pragma unroll
            for (int i = 0; i < TW; i++) {
                if (i + 1 < TW)
#pragma unroll
                    for (int c = 0; c < KC; c++) acc2[(i + 1) & 1][c] = BF_WMM(false, K0 + KC * (i + 1) + c, &oq[8 * c]);
                v4f bo[4];
                load_tile16(pA + C::A_BOUT + 32 * i, g, bo);
                const float sw = pA[C::A_SW + 3 * TW + i];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        x[i][4 * j + k] = x[i][4 * j + k] + (chunk_sum<KC>(acc2[i & 1], 4 * j + k, so) * sw + bo[j][k]);
                pin16(x[i]);
                if (TAPS && a.taps.acc_out)
#pragma unroll
                    for (int c = 0; c < KC; c++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            a.taps.acc_out[((bl * KC + c) * T + t) * D + 32 * (TW * wave + i) + ch(r, g)] = accbits(acc2[i & 1][c], r);
            }
        }
        // the attention-phase parameters are dead: fetch the next layer's
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        dma(wpar + (size_t)lnext * C::PW_FLOATS, pA, C::A_FLOATS, lane);

        // ---- feed-forward --------------------------------------------------------------------------------
        {
            float y[TW][16];
            layernorm(x, pB + C::B_LN2G, pB + C::B_LN2B, y);
            quant_exchange(y, sa, xq, TAPS ? a.taps.qa_ff1 : nullptr, bl);
        }
        double o64[TW][16];   // int8: float64 sums over the k-chunks
        float o32[TW][16];    // e4m3: fp32 sums over the k-tiles
        constexpr int KF = 3 * KC * TW + KC * TW;   // first feed-forward block of the layer
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            constexpr int SBLK = 4 * KC + 2 * TW;   // blocks of one step
            const int k1 = KF + st * SBLK;          // first matmul: four hidden tiles of this wave (half a 256-wide chunk)
            float sh[2];                            // scales of the step's two chunks
            {
                float hf[4][16];
                float am = 0.0f;
                acc_t acc2[2][KC];
#pragma unroll
                for (int c = 0; c < KC; c++) acc2[0][c] = BF_WMM(false, k1 + c, &xq[8 * c]);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if (i + 1 < 4)
#pragma unroll
                        for (int c = 0; c < KC; c++) acc2[(i + 1) & 1][c] = BF_WMM(false, k1 + KC * (i + 1) + c, &xq[8 * c]);
                    v4f b1[4];
                    load_tile16(pB + C::B_BFF1 + 128 * st + 32 * i, g, b1);
                    const float sw = pB[C::B_SW + 4 * st + i];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            const float v = __builtin_fmaxf(chunk_sum<KC>(acc2[i & 1], 4 * j + k, sa) * sw + b1[j][k], 0.0f);
                            hf[i][4 * j + k] = v;
                            am = __builtin_fmaxf(am, v);
                        }
                    pin16(hf[i]);
                    if (TAPS && a.taps.acc_ff1)
#pragma unroll
                        for (int c = 0; c < KC; c++)
#pragma unroll
                            for (int r = 0; r < 16; r++)
                                a.taps.acc_ff1[((bl * KC + c) * T + t) * F + 512 * st + 128 * wave + 32 * i + ch(r, g)] = accbits(acc2[i & 1][c], r);
                }
                // quantiser over the 256-wide chunk this wave shares with its neighbour (waves 0,1: first
                // chunk of the step; 2,3: second).  int8: unsigned, bytes stored as q - 128 for the signed
                // MFMA; e4m3: the ordinary signed quantiser (the values are non-negative)
                xch[2 * 256 + wave * 64 + lane] = am;
                lds_barrier();
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    float m = __builtin_fmaxf(xch[2 * 256 + (2 * c) * 64 + lane], xch[2 * 256 + (2 * c + 1) * 64 + lane]);
                    m = __builtin_fmaxf(m, partner(m, g));
                    sh[c] = m > 0.0f ? m / (FP8 ? 8.0f : 255.0f) : 1.0f;
                }
                const float s8 = wave < 2 ? sh[0] : sh[1];
                const float inv = 1.0f / s8;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    v4i w;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const unsigned u = quant4<FP8>(hf[i][4 * j], hf[i][4 * j + 1], hf[i][4 * j + 2], hf[i][4 * j + 3], s8, inv);
                        if (TAPS && a.taps.qa_ff2)
                            *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl * T + t) * F + 512 * st + 128 * wave + 32 * i + 8 * j + 4 * g) = u;
                        w[j] = (int)(FP8 ? u : (u ^ 0x80808080u));
                    }
                    *reinterpret_cast<v4i*>(hid + (4 * wave + i) * FRAG + lane * 16) = w;
                }
            }
            lds_barrier();
            // second matmul, chunk-major: one chunk of the hidden row (eight fragments) serves this
            // wave's TW output tiles; the float64 sums over the chunks stay in chunk order
            const int k2 = k1 + 4 * KC;
            acc_t acc2[2];
            v4i hqc[8];
#pragma unroll
            for (int s = 0; s < 8; s++) hqc[s] = *reinterpret_cast<const v4i*>(hid + s * FRAG + lane * 16);
            acc2[0] = BF_WMM(false, k2, &hqc[0]);
#pragma unroll
            for (int idx = 0; idx < 2 * TW; idx++) {
                const int c = idx / TW, i = idx % TW;
                v4i ws[4];
                if (!FP8) load_tile16i(pB + C::B_WSUM + (2 * st + c) * CW + 32 * i, g, ws);
                if (idx + 1 < 2 * TW) {
                    if ((idx + 1) % TW == 0)
#pragma unroll
                        for (int s = 0; s < 8; s++)
                            hqc[s] = *reinterpret_cast<const v4i*>(hid + (8 * (c + 1) + s) * FRAG + lane * 16);
                    acc2[(idx + 1) & 1] = BF_WMM(false, k2 + idx + 1, &hqc[0]);
                }
                const acc_t acc = acc2[idx & 1];
                if constexpr (FP8) {
                    // descale each 256-deep tile with its own scales, fp32 sum over the tiles
                    const float sw = pB[C::B_SW + 16 + i * KCF + 2 * st + c];
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const float part = (accf(acc, r) * sh[c]) * sw;
                        o32[i][r] = (st == 0 && c == 0) ? part : o32[i][r] + part;
                        if (TAPS && a.taps.acc_ff2)
                            a.taps.acc_ff2[((bl * KCF + 2 * st + c) * T + t) * D + 32 * (TW * wave + i) + ch(r, g)] = accbits(acc, r);
                    }
                    pin16(o32[i]);
                } else {
                    const double sc = (double)sh[c];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            const int full = accbits(acc, 4 * j + k) + ws[j][k];
                            o64[i][4 * j + k] = (st == 0 && c == 0) ? (double)full * sc
                                                                    : __builtin_fma((double)full, sc, o64[i][4 * j + k]);
                            if (TAPS && a.taps.acc_ff2)
                                a.taps.acc_ff2[((bl * KCF + 2 * st + c) * T + t) * D + 32 * (TW * wave + i) + 8 * j + 4 * g + k] = full;
                        }
#pragma unroll
                    for (int r = 0; r < 16; r++) pin(o64[i][r]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < TW; i++) {
            v4f b2[4];
            load_tile16(pB + C::B_BFF2 + 32 * i, g, b2);
            const float sw = pB[C::B_SW + 16 + i];
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
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        dma(wpar + (size_t)lnext * C::PW_FLOATS + C::A_FLOATS, pB, C::B_FLOATS, lane);
#undef BF_WMM
        if (TAPS && a.taps.resid)
#pragma unroll
            for (int i = 0; i < TW; i++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    a.taps.resid[(bl * T + t) * D + 32 * (TW * wave + i) + ch(r, g)] = x[i][r];
    }

    // ---- final norm and heads --------------------------------------------------------------------------
    // The first head block is in the fragment registers unless a layer range that stops early left
    // the blocks of the next layer there: then restart the stream at the head blocks.
    const int hseq0 = (a.n_layers - a.l0) * BPW;
    wait_vm<0>();   // also: no parameter copy is still landing where the normalised stream goes
    if (a.l1 != a.n_layers) {
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
    float hn[TW][16];
    layernorm(x, gp + C::G_NFG + CW * wave, gp + C::G_NFB + CW * wave, hn);
    if (TAPS && a.taps.normed)
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.normed[((size_t)b * T + t) * D + 32 * (TW * wave + i) + ch(r, g)] = hn[i][r];
    // publish as B-operand fragments (n, j): lane holds the four floats of register quad j
    float* const hnb = reinterpret_cast<float*>(hid);
#pragma unroll
    for (int i = 0; i < TW; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v4f v = {hn[i][4 * j], hn[i][4 * j + 1], hn[i][4 * j + 2], hn[i][4 * j + 3]};
            *reinterpret_cast<v4f*>(hnb + (((TW * wave + i) * 4 + j) * 64 + lane) * 4) = v;
        }
    lds_barrier();
    // wave m multiplies head tile m (rows 32m..32m+31 of [policy; promo; value; 0]) over the whole
    // width, one fused-multiply-add chain in (tile, quad, element) order; wave 3's tile is zero
    v16f head = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (TWIN) {
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

    // value: king token of the side to move, lane half 1 of head tile 2 holds rows 68..70
    if (wave == 2) {
        const int king = ctrl < 0 ? 31 : 15;
        if (lane == 32 + king) {
            float v;
            if (a.n_value == 1) {
                v = tanh_dev(head[0]);
            } else {
                const float r0 = head[0], r1 = head[1], r2 = head[2];
                const float mx = __builtin_fmaxf(__builtin_fmaxf(r0, r1), r2);
                const float e0 = exp_neg(r0 - mx), e1 = exp_neg(r1 - mx), e2 = exp_neg(r2 - mx);
                v = (e2 - e0) / ((e0 + e1) + e2);
            }
            a.value[b] = v;
        }
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
    if (wave < 2) {
        unsigned long long mw = ~0ull;
        if (a.mask) mw = a.mask[(size_t)b * T + t];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int sq = 32 * wave + 8 * j + 4 * g + k;
                const bool legal = (mw >> sq) & 1ull;
                v[k] = legal ? head[4 * j + k] : -__builtin_inff();
                // squares are visited in increasing order within a lane, so '>' keeps the lowest
                if (legal && (bi == 0x7fffffff || v[k] > bv)) { bv = v[k]; bi = t * 64 + sq; }
            }
            const size_t at = ((size_t)b * T + t) * 64 + 32 * wave + 8 * j + 4 * g;
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
        if (lane == 0) {
            xch[wave * 2] = bv;
            xch[wave * 2 + 1] = __int_as_float(bi);
        }
        lds_barrier();
        if (wave == 0 && lane == 0) {
            const float ov = xch[2];
            const int oi = __float_as_int(xch[3]);
            const bool take = (oi != 0x7fffffff) && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
            bi = take ? oi : bi;
            a.best[b] = bi == 0x7fffffff ? -1 : bi;
        }
    }
}

template <int DM, bool TAPS, bool TWIN, bool FP8 = false>
hipError_t launch_board(const KArgs& k, hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be requested once per kernel (per thread: cheap)
    static thread_local bool lds_set = false;
    constexpr int lds_bytes = Cfg<DM, TWIN>::LDS_BYTES;
    if (!lds_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&board_kernel<DM, TAPS, TWIN, FP8>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return e;
        lds_set = true;
    }
    hipLaunchKernelGGL((board_kernel<DM, TAPS, TWIN, FP8>), dim3(k.n), dim3(THREADS), lds_bytes, stream, k);
    return hipGetLastError();
}

}  // namespace board
}  // namespace bf
