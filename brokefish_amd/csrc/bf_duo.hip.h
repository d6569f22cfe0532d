// The evaluator with TWO positions per workgroup of eight wavefronts (256-wide network).
//
// The decomposition is the eight-wavefront form of bf_board.hip.h -- wavefront (q, sub) owns
// tile 2q + sub of the model width, which is also its attention head, half of quarter q's tiles
// in every matmul, and reads its blocks out of the quarter's weight stream where they lie
// (board::block_at) -- but every wavefront does its share for two positions at once.  A weight
// fragment fetched from L2 into registers is then the A operand of two products, one per
// position, so a launch streams the weights once per pair of positions instead of once per
// position, and a wavefront has two independent instruction streams to fill its waits with.
// The quantised activations of both positions stay in LDS and are read as B operands at each
// product; the row statistics of both positions travel through the same exchange and the same
// workgroup barrier.  The arithmetic is that of the other kernels operation for operation, so
// the results are bit-identical to theirs.
//
// NPOS = 1 is the same kernel with one position per workgroup: the latency form for launches of
// at most one workgroup per compute unit (each wavefront one tile of the width, every product
// issued under the previous product's epilogue, and the workgroups of an XCD warming the L2
// with the next layer's weights one layer ahead).
//
// LDS map (bytes): [xch: 3 slots x 2 positions x 8 waves x 64 floats] [hid: the quantised hidden
// row, 32 KiB per position] [act: the quantised row of the width, 8 KiB per position] [par: one
// copy of each quarter's side parameters, shared by its two wavefronts and both positions]
// [tok: the activation scale of every token of the row that feeds QKV, per position].
// During the heads the normalised stream of a position (32 KiB, fp32) overlays its hidden row.
#pragma once

#include "bf_board.hip.h"

// register sets of the weight prefetch (one set = half a block; a set is refilled the moment its
// half-block has been consumed, so all of them are in flight or full between products)
#ifndef BF_DUO_SETS
#define BF_DUO_SETS 3
#endif

namespace bf {
namespace duo {

using board::block_at;
using board::BlockAt;
using board::dma;
using board::frag_mma;
using board::lds;
using board::lds_barrier;
using board::tapbits;
using board::wait_vm;

template <bool FP8, int NP_>
struct Cfg : Layout<256> {
    static constexpr int NP = NP_, NW = 8;   // positions per workgroup (2; 1: the latency form), wavefronts
    static constexpr int XS = NP * NW * 64;               // floats of one exchange slot
    static constexpr int XCH_OFF = 0;
    static constexpr int HID_OFF = XCH_OFF + 3 * XS * 4;
    static constexpr int HID_P = (F / 32) * FRAG;         // a position's hidden row
    static constexpr int ACT_OFF = HID_OFF + NP * HID_P;
    // a position's quantised row of the width: operand bytes; in the e4m3 format widened to fp16 on
    // the way in (every e4m3 value is an fp16 value), so that the products read ready-made operands
    static constexpr int ACT_FRAG = FP8 ? 2 * FRAG : FRAG;
    static constexpr int ACT_P = NT * ACT_FRAG;
    static constexpr int PAR_OFF = ACT_OFF + NP * ACT_P;
    static constexpr int PWL_FLOATS = A_FLOATS + B_FLOATS;
    static constexpr int TOK_OFF = PAR_OFF + 4 * PWL_FLOATS * 4;   // activation scale of every token, per position
    static constexpr int USED_BYTES = TOK_OFF + NP * 32 * 4;
    // The one-position form serves launches of at most one workgroup per compute unit: asking for
    // more than half of a unit's LDS keeps the dispatcher from placing two of them on one unit
    // while another unit stays empty.
    static constexpr int LDS_BYTES = NP == 1 && USED_BYTES < 81 * 1024 ? 81 * 1024 : USED_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget: one workgroup per compute unit");
    static_assert(NT * 4 * FRAG <= HID_P, "normalised stream overlay");
};

// one 16-deep step on operands already widened to fp16; int8 builds never call it
template <bool SWAP>
__device__ __forceinline__ v16f f16_step(const v8h& w, const v8h& act, const v16f& acc) {
    return SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_f16(act, w, acc, 0, 0, 0)
                : __builtin_amdgcn_mfma_f32_32x32x16_f16(w, act, acc, 0, 0, 0);
}
template <bool SWAP>
__device__ __forceinline__ v16i f16_step(const v8h&, const v8h&, const v16i& acc) { return acc; }

template <bool TAPS, bool FP8, bool PROF = false, int NPOS = 2>
__global__ __launch_bounds__(512, 1) void duo_kernel(const KArgs a) {
    typedef Cfg<FP8, NPOS> C;
    static_assert(NPOS == 2 || (NPOS == 1 && !FP8), "one position per workgroup: the int8 format");
    typedef typename Acc<FP8>::type acc_t;
    constexpr int NP = C::NP, D = C::D, F = C::F, NT = C::NT, TW = C::TW, CW = C::CW, KCF = C::KCF;
    constexpr int STEPS = C::STEPS, BPW = C::BPW, HB = C::HB;
    constexpr int NB = BPW / 2;      // weight blocks a wave consumes per layer
    constexpr int HT = 2;            // hidden tiles a wave computes per feed-forward step
    constexpr int NSETS = BF_DUO_SETS;
    constexpr int XS = C::XS, PS = C::NW * 64;   // floats of an exchange slot; of one position's part of it
    constexpr int HALF = BLOCK / 2;
    static_assert(C::KC == 1 && STEPS == TW && KCF == 2 * STEPS, "the 256-wide network");
    static_assert((2 * NB) % NSETS == 0, "register set of a half-block must not depend on the layer");
    static_assert(NSETS - 1 <= 2 * HB + 2, "the first prefetches of the heads stay inside the head blocks");
    static_assert(board::block_at_covers_layer<1, TW, 2, BPW, true>(), "block_at must enumerate a layer's blocks exactly once");

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = wave & 3, sub = wave >> 2;
    const int tile = TW * q + sub;   // the tile of the width (and the head) this wave owns
    const int t = lane & 31, g = lane >> 5;

    // the positions of this workgroup: its own NP slots of the launch, or those entries of the
    // compacted leaf list.  A slot without a position (past the end, skipped, not in this launch)
    // computes its neighbour's position again and stores nothing; a workgroup without any position
    // leaves before the first barrier.
    int bp[NP];
    bool live[NP];
    {
        const int cnt = a.leaf_index ? *a.leaf_count : a.n;
        bool any = false;
        int some = 0;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int j = NP * (int)blockIdx.x + p;
            int b = j;
            bool ok = j < cnt;
            if (a.leaf_index) {
                b = ok ? __builtin_amdgcn_readfirstlane(a.leaf_index[j]) : 0;
                ok = ok && (unsigned)b < (unsigned)a.n;
            }
            if (ok && a.active) ok = a.active[b] != 0;
            bp[p] = ok ? b : 0;
            live[p] = ok;
            if (ok) { any = true; some = b; }
        }
        if (!any) return;
#pragma unroll
        for (int p = 0; p < NP; p++)
            if (!live[p]) bp[p] = some;
    }
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
#ifdef BF_EXP_NOBARRIER   // timing experiment: no workgroup barriers (results are wrong)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#else
            lds_barrier();
#endif
        }
    };

    float* const xch = reinterpret_cast<float*>(lds + C::XCH_OFF);
    uint8_t* const hid = lds + C::HID_OFF;
    uint8_t* const act = lds + C::ACT_OFF;
    float* const tok = reinterpret_cast<float*>(lds + C::TOK_OFF);
    const bool par_owner = sub == 0;
    float* const pA = reinterpret_cast<float*>(lds + C::PAR_OFF) + q * C::PWL_FLOATS;
    float* const pB = pA + C::A_FLOATS;
    const uint8_t* const wsrc =
        a.wstream + ((size_t)q * ((size_t)a.n_layers * BPW + HB + 1) + (size_t)a.l0 * BPW) * BLOCK + lane * 16;
    const float* const wpar = a.fparams + (size_t)q * a.n_layers * C::PW_FLOATS;
    const float* const gp = a.fparams + (size_t)4 * a.n_layers * C::PW_FLOATS;

    // half-block `hseq` of the quarter's stream into register set `set`
    v4i frt[NSETS][4];
    auto load_half = [&](int hseq, int set) {
#ifdef BF_EXP_SAMEBLOCK   // timing experiment: every load reads the wave's first half-block (an L1 hit)
        const uint8_t* src = wsrc + (size_t)(hseq & 0) * HALF;
#else
        const uint8_t* src = wsrc + (size_t)hseq * HALF;
#endif
#ifdef BF_EXP_NOLOAD   // timing experiment: no weight traffic
        (void)src;
#pragma unroll
        for (int s = 0; s < 4; s++) asm volatile("" : "=v"(frt[set][s]));
#else
#pragma unroll
        for (int s = 0; s < 4; s++) frt[set][s] = *reinterpret_cast<const v4i*>(src + s * FRAG);
#endif
    };
    // the wave's hh-th half-block of the layer whose stream starts at block `base` (hh may run into
    // the following layer, whose stream starts at block `next`)
    auto fetch_half = [&](int hh, int base, int next) {
        const int n = hh / 2;
        const BlockAt at = block_at<1, TW, 2, true>(n % NB);
        load_half(2 * ((n < NB ? base : next) + at.a + sub * at.b) + hh % 2, hh % NSETS);
    };

    // L2 warm-up for launches of one wave of workgroups (NP == 1): such a launch moves through the
    // layers in step, so every first touch of a weight line would be an L2 miss that all the
    // workgroups behind that L2 wait for.  The workgroups of an XCD (dispatched round-robin, so
    // blockIdx / 8 numbers them) each touch a share of the lines of a layer's blocks one layer ahead,
    // one dword per 128-byte line; the values are never used.  A hint only: a share that nobody
    // touches (workgroups that left early, another dispatch order) costs time, not correctness.
    // Below four workgroups per XCD the touches cover too little to pay for the loads they delay
    // (loads return in order), above one workgroup per compute unit the launch is not in step.
#ifdef BF_EXP_NOWARM   // timing experiment: no warm-up touches (results stay right)
    constexpr int WARM = 0;
#else
    constexpr int WARM = NP == 1 ? 2 : 0;
#endif
    constexpr int LAYER_LINES = BPW * BLOCK / 128;   // per quarter
    int warm[WARM > 0 ? WARM : 1] = {};
    auto warm_l2 = [&](int blk0) {
        if constexpr (WARM > 0) {
            const int per = ((int)gridDim.x + 7) >> 3;
#pragma unroll
            for (int j = 0; j < WARM; j++) {
                const int line = ((j * per + ((int)blockIdx.x >> 3)) * 8 + wave) * 64 + lane;
                if (line < 4 * LAYER_LINES && gridDim.x > 24 && gridDim.x <= 256) {
                    const int qq = line / LAYER_LINES, off = line % LAYER_LINES;
                    warm[j] = *reinterpret_cast<const int*>(
                        a.wstream + ((size_t)qq * ((size_t)a.n_layers * BPW + HB + 1) + (size_t)blk0) * BLOCK + (size_t)off * 128);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto warm_done = [&]() {   // the touches have long returned: retire their registers
        if constexpr (WARM > 0) {
#pragma unroll
            for (int j = 0; j < WARM; j++) asm volatile("" ::"v"(warm[j]));
        }
    };

    // Row sum over the width for both positions: a wave's 16 values form one chain from zero, the
    // two tile sums of a quarter are added, then the four quarter sums in order.  One exchange slot
    // per call site, so that a fast wave's next partial cannot overwrite what a slow wave still
    // reads: between two uses of a slot lies at least one other workgroup barrier.
    auto xsum2 = [&](const float (&part)[NP], int slot, float (&out)[NP]) {
#pragma unroll
        for (int p = 0; p < NP; p++) xch[slot * XS + p * PS + wave * 64 + lane] = part[p];
        barrier();
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const float* s = xch + slot * XS + p * PS + lane;
            out[p] = (((s[0] + s[256]) + (s[64] + s[320])) + (s[128] + s[384])) + (s[192] + s[448]);
        }
    };
    auto layernorm2 = [&](const float (&x)[NP][16], const float* gamma, const float* beta, float (&y)[NP][16]) {
        float part[NP], s[NP], mean[NP], v[NP], rstd[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) acc = acc + x[p][r];
            part[p] = acc;
        }
        xsum2(part, 0, s);
#pragma unroll
        for (int p = 0; p < NP; p++) {
            mean[p] = (s[p] + partner(s[p], g)) * (1.0f / D);
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float d = x[p][r] - mean[p];
                acc = __builtin_fmaf(d, d, acc);
            }
            part[p] = acc;
        }
        xsum2(part, 1, v);
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const float var = (v[p] + partner(v[p], g)) * (1.0f / D);
            rstd[p] = 1.0f / __builtin_sqrtf(var + a.eps);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v4f ga = ldg4(gamma + 8 * j + 4 * g);
            const v4f be = ldg4(beta + 8 * j + 4 * g);
#pragma unroll
            for (int p = 0; p < NP; p++)
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float d = x[p][4 * j + k] - mean[p];
                    y[p][4 * j + k] = __builtin_fmaf(d * rstd[p], ga[k], be[k]);
                }
        }
    };
    // signed quantiser of both positions' rows: one scale per row; this wave's bytes go to the
    // position's activation buffer, from which every wave reads its B operands
    auto quant_exchange2 = [&](const float (&y)[NP][16], float (&sa)[NP], int8_t* tap, const size_t (&tap_row)[NP], bool publish_scales) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            float am = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) am = __builtin_fmaxf(am, __builtin_fabsf(y[p][r]));
            xch[2 * XS + p * PS + wave * 64 + lane] = am;
        }
        barrier();
#pragma unroll
        for (int p = 0; p < NP; p++) {
            float m = 0.0f;
#pragma unroll
            for (int w = 0; w < C::NW; w++) m = __builtin_fmaxf(m, xch[2 * XS + p * PS + w * 64 + lane]);
            m = __builtin_fmaxf(m, partner(m, g));
            sa[p] = m > 0.0f ? (FP8 ? m * 0.125f : div127(m)) : 1.0f;
            if (publish_scales && wave == 0 && g == 0) tok[p * 32 + t] = sa[p];
            const float inv = 1.0f / sa[p];
            v4i w;
#pragma unroll
            for (int j = 0; j < 4; j++)
                w[j] = (int)quant4<FP8>(y[p][4 * j], y[p][4 * j + 1], y[p][4 * j + 2], y[p][4 * j + 3], sa[p], inv);
            if constexpr (FP8) {
                const v2l wl = __builtin_bit_cast(v2l, w);
#pragma unroll
                for (int h = 0; h < 2; h++)
                    *reinterpret_cast<v8h*>(act + p * C::ACT_P + (2 * tile + h) * FRAG + lane * 16) = e4m3x8_as_f16(wl[h]);
            } else {
                *reinterpret_cast<v4i*>(act + p * C::ACT_P + tile * FRAG + lane * 16) = w;
            }
            if (TAPS && tap && live[p])
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(tap + (tap_row[p] * T + t) * D + 32 * tile + 8 * j + 4 * g) = w[j];
        }
        barrier();
    };
    const uint8_t* const act0 = act + lane * 16;
    const uint8_t* const hid0 = hid + lane * 16;
    auto ldsfrag = [&](const uint8_t* p) -> v4i { return *reinterpret_cast<const v4i*>(p); };

    // ---- start the weight stream and the first layer's parameters --------------------------------
    if (nl_run > 0) {
#pragma unroll
        for (int j = 0; j < NSETS; j++) fetch_half(j, 0, BPW);
        warm_l2(a.l0 * BPW);
        if (par_owner) {
            dma(wpar + (size_t)a.l0 * C::PW_FLOATS, pA, C::A_FLOATS, lane);
            dma(wpar + (size_t)a.l0 * C::PW_FLOATS + C::A_FLOATS, pB, C::B_FLOATS, lane);
        }
    }

    // An encoder-only launch (tap table with `alive`): the residual stream comes in through x_in, the
    // token mask through `alive`, the stream after the last layer goes out through resid_last, and
    // there are no board words and no heads.
    const bool enc_only = TAPS && a.taps.alive != nullptr;
    // ---- embedding (this wave's tile, both positions) ----------------------------------------------
    float x[NP][16];
    unsigned alive[NP];
    int ctrl[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        const int b = bp[p];
        const unsigned word = enc_only ? (a.taps.alive[(size_t)b * T + t] ? 0u : 0x800u) : a.boards[(size_t)b * T + t];
        ctrl[p] = enc_only ? 1 : a.control[b];
        alive[p] = (unsigned)__ballot(((word >> 11) & 1) == 0 && g == 0);
        if (TAPS && a.taps.x_in) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = ldg4(a.taps.x_in + ((size_t)b * T + t) * D + 32 * tile + 8 * j + 4 * g);
#pragma unroll
                for (int k = 0; k < 4; k++) x[p][4 * j + k] = v[k];
            }
        } else {
            const int stm = ctrl[p] < 0;
            int clock = (ctrl[p] < 0 ? -ctrl[p] : ctrl[p]) - 1;
            clock = clock < 0 ? 0 : (clock > 100 ? 100 : clock);
            int rp = a.rep[b];
            rp = rp > 2 ? 2 : rp;
            int ts = ((word >> 6) & 7) * 2 + ((word >> 9) & 1);
            ts = ts > 11 ? 11 : ts;
            const int ct = ((word >> 10) & 1) * 2 + stm;
            const int own = 32 * tile + 4 * g;
            const float* e_sq = gp + C::G_SQ + (word & 63) * D + own;
            const float* e_ts = gp + C::G_TS + ts * D + own;
            const float* e_ct = gp + C::G_CT + ct * D + own;
            const float* e_ck = gp + C::G_CLOCK + clock * D + own;
            const float* e_rp = gp + C::G_REP + rp * D + own;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = 8 * j;
                const v4f vs = ldg4(e_sq + c), vt = ldg4(e_ts + c), vc = ldg4(e_ct + c);
                const v4f vk = ldg4(e_ck + c), vr = ldg4(e_rp + c);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float per_board = vk[k] + vr[k];
                    float v = vs[k] + vt[k];
                    v = v + vc[k];
                    x[p][4 * j + k] = v + per_board;
                }
            }
        }
        if (TAPS && a.taps.embed && live[p])
#pragma unroll
            for (int r = 0; r < 16; r++) a.taps.embed[((size_t)b * T + t) * D + 32 * tile + ch(r, g)] = x[p][r];
    }

    wait_vm<0>();   // the parameters have landed (published to the quarter's other wave by the next barrier)
    warm_done();
    BF_PHASE(PH_EMBED);

    for (int l = a.l0; l < a.l1; l++) {
        const int li = l - a.l0;
        size_t bl[NP];   // tap rows
#pragma unroll
        for (int p = 0; p < NP; p++) bl[p] = (size_t)bp[p] * nl_run + li;
        const int lnext = l + 1 < a.l1 ? l + 1 : l;   // after the last layer the same layer is fetched again (and never used)
#ifdef BF_EXP_SAMELAYER   // timing experiment: every layer streams the first layer's blocks (they stay in L2)
        const int lbase = 0 * li, lfollow = 0 * lnext;
#else
        const int lbase = li * BPW, lfollow = (lnext - a.l0) * BPW;
#endif
        // One position's product with the wave's k-th block of this layer: eight 32-deep steps against
        // the operand row whose fragment 0 is at BSRC (lane offset included), each fragment fetched
        // from LDS one step ahead.  The block's two halves sit in register sets 2k % NSETS and
        // (2k + 1) % NSETS; the last position refills each of them as soon as it has consumed it (with
        // the half-blocks NSETS on), so every set is in flight or full across the phases between
        // products (attention, the LayerNorms).
        // BETWEEN(s) runs after step s has been issued: an eighth of the previous product's epilogue,
        // which the vector ALU works through while the matrix pipe runs; nothing is scheduled across
        // the end of a step.
#ifndef BF_DUO_AHEAD
#define BF_DUO_AHEAD 1   // steps between the LDS fetch of an operand fragment and its use
#endif
#define BF_DUO_CHAIN(SWAP, k, p, BSRC, INIT, R, BETWEEN)                                             \
    do {                                                                                             \
        constexpr int A_ = BF_DUO_AHEAD;                                                             \
        const uint8_t* const b_ = (BSRC);                                                            \
        v4i ring_[A_ + 1];                                                                           \
        _Pragma("unroll") for (int u_ = 0; u_ < A_; u_++) ring_[u_] = ldsfrag(b_ + u_ * FRAG);       \
        (R) = (INIT);                                                                                \
        _Pragma("unroll") for (int s_ = 0; s_ < 8; s_++) {                                           \
            if (s_ + A_ < 8) ring_[(s_ + A_) % (A_ + 1)] = ldsfrag(b_ + (s_ + A_) * FRAG);           \
            (R) = frag_mma<SWAP>(frt[(2 * (k) + s_ / 4) % NSETS][s_ % 4], ring_[s_ % (A_ + 1)], (R)); \
            BETWEEN(s_);                                                                             \
            __builtin_amdgcn_sched_barrier(0);                                                       \
            if ((p) == NP - 1 && s_ == 3) fetch_half(2 * (k) + NSETS, lbase, lfollow);               \
        }                                                                                            \
        if ((p) == NP - 1) fetch_half(2 * (k) + NSETS + 1, lbase, lfollow);                          \
    } while (0)
        // e4m3: both positions' products with the wave's k-th block, step by step.  A weight fragment is
        // widened to fp16 once and multiplied with both positions' operands; these come from LDS
        // already widened (A16: the row of the width) or as bytes (the hidden row).  Each accumulator
        // sees its sixteen 16-deep steps in order, as in the other kernels.
#define BF_DUO_PAIR_F8(SWAP, k, A16, B0, B1, R)                                                      \
    do {                                                                                             \
        const uint8_t* const bp_[2] = {(B0), (B1)};                                                  \
        (R)[0] = zero;                                                                               \
        (R)[1] = zero;                                                                               \
        /* the operands of a step are fetched from LDS one step ahead: [position][half] */           \
        v4i cur_[2][2], nxt_[2][2];                                                                  \
        _Pragma("unroll") for (int p_ = 0; p_ < 2; p_++)                                             \
            _Pragma("unroll") for (int h_ = 0; h_ < ((A16) ? 2 : 1); h_++)                           \
                cur_[p_][h_] = ldsfrag(bp_[p_] + ((A16) ? h_ : 0) * FRAG);                           \
        _Pragma("unroll") for (int s_ = 0; s_ < 8; s_++) {                                           \
            _Pragma("unroll") for (int p_ = 0; p_ < 2; p_++)                                         \
                _Pragma("unroll") for (int h_ = 0; h_ < ((A16) ? 2 : 1); h_++)                       \
                    nxt_[p_][h_] = s_ + 1 < 8 ? ldsfrag(bp_[p_] + ((A16) ? 2 * (s_ + 1) + h_ : s_ + 1) * FRAG) : cur_[p_][h_]; \
            const v2l wl_ = __builtin_bit_cast(v2l, frt[(2 * (k) + s_ / 4) % NSETS][s_ % 4]);        \
            _Pragma("unroll") for (int h_ = 0; h_ < 2; h_++) {                                       \
                const v8h wh_ = e4m3x8_as_f16(wl_[h_]);                                              \
                _Pragma("unroll") for (int p_ = 0; p_ < 2; p_++) {                                   \
                    v8h ah_;                                                                         \
                    if (A16) ah_ = __builtin_bit_cast(v8h, cur_[p_][h_]);                            \
                    else ah_ = e4m3x8_as_f16(__builtin_bit_cast(v2l, cur_[p_][0])[h_]);              \
                    (R)[p_] = f16_step<SWAP>(wh_, ah_, (R)[p_]);                                     \
                }                                                                                    \
            }                                                                                        \
            __builtin_amdgcn_sched_barrier(0);                                                       \
            _Pragma("unroll") for (int p_ = 0; p_ < 2; p_++)                                         \
                _Pragma("unroll") for (int h_ = 0; h_ < ((A16) ? 2 : 1); h_++) cur_[p_][h_] = nxt_[p_][h_]; \
            if (s_ == 3) fetch_half(2 * (k) + NSETS, lbase, lfollow);                                \
        }                                                                                            \
        fetch_half(2 * (k) + NSETS + 1, lbase, lfollow);                                             \
    } while (0)
        const acc_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        auto none = [&](int) {};
        const uint8_t* const act1 = act0 + C::ACT_P;

        // ---- LayerNorm 1, quantise, exchange -----------------------------------------------------------
        float sa[NP];
        {
            float y[NP][16];
            layernorm2(x, pA + C::A_LN1G + 32 * sub, pA + C::A_LN1B + 32 * sub, y);
            quant_exchange2(y, sa, TAPS ? a.taps.qa_qkv : nullptr, bl, true);
        }
        // the quarter's feed-forward parameters of this layer (the first layer's came with the start)
        if (par_owner && li > 0) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)l * C::PW_FLOATS + C::A_FLOATS, pB, C::B_FLOATS, lane);
        }
        BF_PHASE(PH_LN1);

        // ---- attention: this wave's head, both positions ------------------------------------------------
        float o[NP][16];
        {
            float qf[NP][16], kf[NP][16], vf[NP][16];
            const float swq = pA[C::A_SW + sub], swk = pA[C::A_SW + TW + sub], swv = pA[C::A_SW + 2 * TW + sub];
            const float bv = pA[C::A_BV + 32 * sub + t];
            acc_t acc[2];   // product n of a sequence uses accumulator n & 1; the previous one's epilogue runs under it
            v4f bq[4], bk[4], stok[NP][4];
            // the epilogues, two accumulator registers at a time (slice s of eight)
            auto epi_q = [&](int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    qf[p][e] = accf(acc[ai], e) * sa[p] * swq + bq[e / 4][e % 4];
                    if (TAPS && a.taps.acc_qkv && live[p])
                        a.taps.acc_qkv[(bl[p] * T + t) * 3 * D + 32 * tile + ch(e, g)] = tapbits<false>(acc[ai], e);
                }
            };
            auto epi_k = [&](int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    kf[p][e] = accf(acc[ai], e) * sa[p] * swk + bk[e / 4][e % 4];
                    if (TAPS && a.taps.acc_qkv && live[p])
                        a.taps.acc_qkv[(bl[p] * T + t) * 3 * D + D + 32 * tile + ch(e, g)] = tapbits<false>(acc[ai], e);
                }
            };
            // V tile: rows are tokens, so the activation scale is that of token ch(e, g)
            auto epi_v = [&](int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    vf[p][e] = accf(acc[ai], e) * stok[p][e / 4][e % 4] * swv + bv;
                    if (TAPS && a.taps.acc_qkv && live[p])
                        a.taps.acc_qkv[(bl[p] * T + ch(e, g)) * 3 * D + 2 * D + 32 * tile + t] = tapbits<false>(acc[ai], e);
                }
            };
            auto epi_qkv = [&](int tq, int p, int s, int ai) {
                if (tq == 0) epi_q(p, s, ai);
                else if (tq == 1) epi_k(p, s, ai);
                else epi_v(p, s, ai);
            };
            load_tile16(pA + C::A_BQ + 32 * sub, g, bq);
            if constexpr (FP8) {
                // e4m3: a block's two products share the widening of its weight fragments, the
                // epilogues of both positions follow
                BF_DUO_PAIR_F8(false, 0, true, act0, act1, acc);
#pragma unroll
                for (int s = 0; s < 8; s++) { epi_q(0, s, 0); epi_q(1, s, 1); }
                load_tile16(pA + C::A_BK + 32 * sub, g, bk);
                BF_DUO_PAIR_F8(false, 1, true, act0, act1, acc);
#pragma unroll
                for (int s = 0; s < 8; s++) { epi_k(0, s, 0); epi_k(1, s, 1); }
                load_tile16(tok, g, stok[0]);
                load_tile16(tok + 32, g, stok[1]);
                BF_DUO_PAIR_F8(true, 2, true, act0, act1, acc);
#pragma unroll
                for (int s = 0; s < 8; s++) { epi_v(0, s, 0); epi_v(1, s, 1); }
            } else {
                // Q, K, V blocks in turn, each for every position: 3 NP products
#pragma unroll
                for (int n = 0; n < 3 * NP; n++) {
                    const int tq = n / NP, p = n % NP;
                    if (n == NP) load_tile16(pA + C::A_BK + 32 * sub, g, bk);
                    if (tq == 2) load_tile16(tok + 32 * p, g, stok[p]);
                    auto between = [&](int s) {
                        if (n > 0) epi_qkv((n - 1) / NP, (n - 1) % NP, s, (n - 1) & 1);
                    };
                    if (tq == 2) BF_DUO_CHAIN(true, 2, p, act0 + p * C::ACT_P, zero, acc[n & 1], between);
                    else BF_DUO_CHAIN(false, tq, p, act0 + p * C::ACT_P, zero, acc[n & 1], between);
                }
#pragma unroll
                for (int s = 0; s < 8; s++) epi_v(NP - 1, s, (3 * NP - 1) & 1);
            }
            BF_PHASE(PH_QKV);
            if (l + 1 < a.l1) warm_l2((l + 1) * BPW);   // the sets are full and the next weight wait is an attention away
#pragma unroll
            for (int p = 0; p < NP; p++) {
                // scores, transposed: lane = query token, register r = key ch(r, g)
                v16f sc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int r = 0; r < 16; r++) sc = BF_F32MMA(kf[p][r], qf[p][r], sc);
                float pr[16];
                float mx = -__builtin_inff();
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float s = sc[r] * 0.17677669529663687f;
                    s = ((alive[p] >> ch(r, g)) & 1u) ? s : -__builtin_inff();
                    pr[r] = s;
                    mx = __builtin_fmaxf(mx, s);
                }
                mx = __builtin_fmaxf(mx, partner(mx, g));
                float lsum = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    pr[r] = exp_neg(pr[r] - mx);
                    lsum = lsum + pr[r];
                }
                const float rl = 1.0f / (lsum + partner(lsum, g));
                v16f oa = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int r = 0; r < 16; r++) oa = BF_F32MMA(vf[p][r], pr[r] * rl, oa);
#pragma unroll
                for (int r = 0; r < 16; r++) o[p][r] = oa[r];
                pin16(o[p]);
            }
            BF_PHASE(PH_ATTN);
        }

        // ---- output projection + residual (this wave's tile) --------------------------------------------
        {
            float so[NP];
            quant_exchange2(o, so, TAPS ? a.taps.qa_out : nullptr, bl, false);
            acc_t acc[2];
            v4f bo[4];
            load_tile16(pA + C::A_BOUT + 32 * sub, g, bo);
            const float sw = pA[C::A_SW + 3 * TW + sub];
            auto epi_o = [&](int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    x[p][e] = x[p][e] + (accf(acc[ai], e) * so[p] * sw + bo[e / 4][e % 4]);
                    if (TAPS && a.taps.acc_out && live[p])
                        a.taps.acc_out[(bl[p] * T + t) * D + 32 * tile + ch(e, g)] = tapbits<false>(acc[ai], e);
                }
            };
            if constexpr (FP8) {
                BF_DUO_PAIR_F8(false, 3, true, act0, act1, acc);
#pragma unroll
                for (int s = 0; s < 8; s++) epi_o(0, s, 0);
            } else {
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    auto between = [&](int s) {
                        if (p > 0) epi_o(p - 1, s, (p - 1) & 1);
                    };
                    BF_DUO_CHAIN(false, 3, p, act0 + p * C::ACT_P, zero, acc[p & 1], between);
                }
            }
#pragma unroll
            for (int s = 0; s < 8; s++) epi_o(NP - 1, s, (NP - 1) & 1);
        }
        BF_PHASE(PH_OUT);

        // ---- feed-forward ---------------------------------------------------------------------------------
        {
            float y[NP][16];
            layernorm2(x, pB + C::B_LN2G + 32 * sub, pB + C::B_LN2B + 32 * sub, y);
            quant_exchange2(y, sa, TAPS ? a.taps.qa_ff1 : nullptr, bl, false);
        }
        // the attention-phase parameters are dead for both waves of the quarter: fetch the next layer's
        if (par_owner) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            dma(wpar + (size_t)lnext * C::PW_FLOATS, pA, C::A_FLOATS, lane);
        }
        BF_PHASE(PH_LN2);
        // First matmul, step by step: each step's two 256-wide chunks are quantised as soon as the step
        // is complete (a chunk spans a pair of quarters); the whole quantised hidden row of both
        // positions stays in LDS.  int8: unsigned, bytes stored as q - 128 for the signed MFMA.
        float sh[NP][KCF];
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            float hf[NP][HT][16];
            float am[NP];
#pragma unroll
            for (int p = 0; p < NP; p++) am[p] = 0.0f;
            acc_t acc[2];
            v4f b1[HT][4];
            float sw1[HT];
            auto epi_f = [&](int i, int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    // int8: the ReLU is the saturation of the unsigned quantiser below, and the
                    // running maximum starts at 0, so negative values need no clamp here
                    float v = accf(acc[ai], e) * sa[p] * sw1[i] + b1[i][e / 4][e % 4];
                    if constexpr (FP8) v = __builtin_fmaxf(v, 0.0f);
                    hf[p][i][e] = v;
                    am[p] = __builtin_fmaxf(am[p], v);
                    if (TAPS && a.taps.acc_ff1 && live[p])
                        a.taps.acc_ff1[(bl[p] * T + t) * F + 512 * st + 128 * q + 32 * (HT * sub + i) + ch(e, g)] = tapbits<false>(acc[ai], e);
                }
            };
#pragma unroll
            for (int i = 0; i < HT; i++) {
                load_tile16(pB + C::B_BFF1 + 128 * st + 32 * (HT * sub + i), g, b1[i]);
                sw1[i] = pB[C::B_SW + 4 * st + HT * sub + i];
                if constexpr (FP8) {
                    BF_DUO_PAIR_F8(false, 4 + HT * st + i, true, act0, act1, acc);
#pragma unroll
                    for (int s = 0; s < 8; s++) { epi_f(i, 0, s, 0); epi_f(i, 1, s, 1); }
                } else {
#pragma unroll
                    for (int p = 0; p < NP; p++) {
                        const int n = NP * i + p;   // product number within the step; the previous one's epilogue runs under it
                        auto between = [&](int s) {
                            if (n > 0) epi_f((n - 1) / NP, (n - 1) % NP, s, (n - 1) & 1);
                        };
                        BF_DUO_CHAIN(false, 4 + HT * st + i, p, act0 + p * C::ACT_P, zero, acc[n & 1], between);
                    }
                }
            }
            if constexpr (!FP8)
#pragma unroll
                for (int s = 0; s < 8; s++) epi_f(HT - 1, NP - 1, s, (NP * HT - 1) & 1);
            // the maxima of consecutive steps go through different exchange slots
            const int xs = (st & 1) ? 0 : 2 * XS;
#pragma unroll
            for (int p = 0; p < NP; p++) xch[xs + p * PS + wave * 64 + lane] = am[p];
            barrier();
#pragma unroll
            for (int p = 0; p < NP; p++) {
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    float m = 0.0f;   // hidden values are >= 0
#pragma unroll
                    for (int u = 0; u < 2; u++)
                        m = __builtin_fmaxf(m, __builtin_fmaxf(xch[xs + p * PS + (2 * c + 4 * u) * 64 + lane],
                                                               xch[xs + p * PS + (2 * c + 1 + 4 * u) * 64 + lane]));
                    m = __builtin_fmaxf(m, partner(m, g));
                    sh[p][2 * st + c] = m > 0.0f ? (FP8 ? m * 0.125f : div255(m)) : 1.0f;
                }
                const float s8 = q < 2 ? sh[p][2 * st] : sh[p][2 * st + 1];
                const float inv = 1.0f / s8;
#pragma unroll
                for (int i = 0; i < HT; i++) {
                    v4i w;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        unsigned u;
                        if constexpr (FP8) u = quant4<true>(hf[p][i][4 * j], hf[p][i][4 * j + 1], hf[p][i][4 * j + 2], hf[p][i][4 * j + 3], s8, inv);
                        else u = quant4_relu_u8(hf[p][i][4 * j], hf[p][i][4 * j + 1], hf[p][i][4 * j + 2], hf[p][i][4 * j + 3], s8, inv);
                        if (TAPS && a.taps.qa_ff2 && live[p])
                            *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl[p] * T + t) * F + 512 * st + 128 * q + 32 * (HT * sub + i) + 8 * j + 4 * g) = u;
                        w[j] = (int)(FP8 ? u : (u ^ 0x80808080u));
                    }
                    *reinterpret_cast<v4i*>(hid + p * C::HID_P + (16 * st + 4 * q + HT * sub + i) * FRAG + lane * 16) = w;
                }
            }
        }
        barrier();   // the whole hidden row of both positions is in LDS
        BF_PHASE(PH_FF1);
        // Second matmul: this wave's output tile over the KCF k-chunks in turn; each chunk's block
        // serves both positions.  int8: the accumulator starts at 128 * sum(w), the offset of the
        // unsigned bytes stored as q - 128; the sums over the chunks are float64 (e4m3: fp32).
        {
            double o64[NP][16];
            float o32[NP][16];
            acc_t acc[2];
            acc_t init = zero;
            float sw2[KCF];   // e4m3: one weight scale per k-chunk
            if constexpr (FP8)
#pragma unroll
                for (int cc = 0; cc < KCF; cc++) sw2[cc] = pB[C::B_SW + 16 + sub * KCF + cc];
            auto epi_2 = [&](int cc, int p, int s, int ai) {
#pragma unroll
                for (int e = 2 * s; e < 2 * s + 2; e++) {
                    if constexpr (FP8) {
                        const float part = (accf(acc[ai], e) * sh[p][cc]) * sw2[cc];
                        o32[p][e] = cc == 0 ? part : o32[p][e] + part;
                    } else {
                        const double sc = (double)sh[p][cc];
                        const int full = accbits(acc[ai], e);
                        o64[p][e] = cc == 0 ? (double)full * sc : __builtin_fma((double)full, sc, o64[p][e]);
                    }
                    if (TAPS && a.taps.acc_ff2 && live[p])
                        a.taps.acc_ff2[((bl[p] * KCF + cc) * T + t) * D + 32 * tile + ch(e, g)] = accbits(acc[ai], e);
                }
            };
#pragma unroll
            for (int cc = 0; cc < KCF; cc++) {
                if constexpr (FP8) {
                    BF_DUO_PAIR_F8(false, 4 + HT * STEPS + cc, false, hid0 + 8 * cc * FRAG, hid0 + C::HID_P + 8 * cc * FRAG, acc);
#pragma unroll
                    for (int s = 0; s < 8; s++) { epi_2(cc, 0, s, 0); epi_2(cc, 1, s, 1); }
                } else {
#pragma unroll
                    for (int p = 0; p < NP; p++) {
                        const int n = NP * cc + p;
                        if (p == 0) {
                            v4i w0[4];
                            load_tile16i(pB + C::B_WSUM + cc * CW + 32 * sub, g, w0);
#pragma unroll
                            for (int j = 0; j < 4; j++)
#pragma unroll
                                for (int k = 0; k < 4; k++) init[4 * j + k] = w0[j][k];
                        }
                        auto between = [&](int s) {
                            if (n > 0) epi_2((n - 1) / NP, (n - 1) % NP, s, (n - 1) & 1);
                        };
                        BF_DUO_CHAIN(false, 4 + HT * STEPS + cc, p, hid0 + p * C::HID_P + 8 * cc * FRAG, init, acc[n & 1], between);
                    }
                }
            }
            if constexpr (!FP8)
#pragma unroll
                for (int s = 0; s < 8; s++) epi_2(KCF - 1, NP - 1, s, (NP * KCF - 1) & 1);
            v4f b2[4];
            load_tile16(pB + C::B_BFF2 + 32 * sub, g, b2);
            const float sw = pB[C::B_SW + 16 + sub];
#pragma unroll
            for (int p = 0; p < NP; p++) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        float upd;
                        if constexpr (FP8) upd = o32[p][4 * j + k] + b2[j][k];
                        else upd = (float)o64[p][4 * j + k] * sw + b2[j][k];
                        x[p][4 * j + k] = x[p][4 * j + k] + upd;
                    }
                pin16(x[p]);
            }
        }
        BF_PHASE(PH_FF2);
        warm_done();
#undef BF_DUO_CHAIN
#undef BF_DUO_PAIR_F8
        if (TAPS && a.taps.resid)
#pragma unroll
            for (int p = 0; p < NP; p++)
                if (live[p])
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.resid[(bl[p] * T + t) * D + 32 * tile + ch(r, g)] = x[p][r];
    }
    if (TAPS && a.taps.resid_last)
#pragma unroll
        for (int p = 0; p < NP; p++)
            if (live[p])
#pragma unroll
                for (int r = 0; r < 16; r++)
                    a.taps.resid_last[((size_t)bp[p] * T + t) * D + 32 * tile + ch(r, g)] = x[p][r];
    if (enc_only) return;   // the same for every wave of the launch

    // ---- final norm and heads --------------------------------------------------------------------------
    // The weight stream is restarted at the head blocks (after the last layer the prefetch ran on
    // into a layer that is not used).
    const int hseq0 = (a.n_layers - a.l0) * BPW;
    wait_vm<0>();   // also: no parameter copy is still landing
#pragma unroll
    for (int j = 0; j < NSETS - 1; j++) load_half(2 * hseq0 + j, j);
    float hn[NP][16];
    layernorm2(x, gp + C::G_NFG + 32 * tile, gp + C::G_NFB + 32 * tile, hn);
    // publish as B-operand fragments (n, j): lane holds the four floats of register quad j
#pragma unroll
    for (int p = 0; p < NP; p++) {
        float* const hnb = reinterpret_cast<float*>(hid + p * C::HID_P);
        if (TAPS && a.taps.normed && live[p])
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.normed[((size_t)bp[p] * T + t) * D + 32 * tile + ch(r, g)] = hn[p][r];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v4f v = {hn[p][4 * j], hn[p][4 * j + 1], hn[p][4 * j + 2], hn[p][4 * j + 3]};
            *reinterpret_cast<v4f*>(hnb + ((tile * 4 + j) * 64 + lane) * 4) = v;
        }
    }
    barrier();
    // Wave (m, p) multiplies head tile m (rows 32m..32m+31 of [policy; promo; value; 0]) with the
    // normalised stream of position p over the whole width, one fused-multiply-add chain in (tile,
    // quad, element) order; quarter 3's tile is zero and stores nothing, so it is not computed.
    // With one position per workgroup the second wave of a quarter has nothing to do here but
    // meet the barriers.
    const int mine = NP == 2 ? sub : 0;   // the position whose heads this wave computes
    const bool heads_here = NP == 2 || sub == 0;
    const float* const hnb = reinterpret_cast<const float*>(hid + mine * C::HID_P);
    v16f head = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if (q < 3 && heads_here) {
#pragma unroll
        for (int hi = 0; hi < 2 * HB; hi++) {
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
    }
    BF_PHASE(PH_HEADS);
    const int b = mine ? bp[NP - 1] : bp[0];
    const bool store = heads_here && (mine ? live[NP - 1] : live[0]);
    const int ctrl_m = mine ? ctrl[NP - 1] : ctrl[0];
    auto value_of = [&](const v16f& hd) -> float {
        if (a.n_value == 1) return tanh_dev(hd[0]);
        const float r0 = hd[0], r1 = hd[1], r2 = hd[2];   // classes loss, draw, win
        const float mx = __builtin_fmaxf(__builtin_fmaxf(r0, r1), r2);
        const float e0 = exp_neg(r0 - mx), e1 = exp_neg(r1 - mx), e2 = exp_neg(r2 - mx);
        return (e2 - e0) / ((e0 + e1) + e2);
    };
    // value (king head): king token of the side to move, lane half 1 of head tile 2 holds rows 68..70
    if (q == 2 && store) {
        const int king = ctrl_m < 0 ? 31 : 15;
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
    // policy (quarters 0 and 1: squares 0..31 and 32..63), optional legal-move AND and argmax
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    if (q < 2 && heads_here) {
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
            if (store) {
                if (a.out_fp32) {
                    const v4f vv = {v[0], v[1], v[2], v[3]};
                    *reinterpret_cast<v4f*>((float*)a.policy + at) = vv;
                } else {
                    const v4h vv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                    *reinterpret_cast<v4h*>((_Float16*)a.policy + at) = vv;
                }
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
        // the two policy waves' winners of a position meet in the exchange slot no row sum uses
        if (q < 2 && heads_here && lane == 0) {
            xch[2 * XS + mine * 4 + q * 2] = bv;
            xch[2 * XS + mine * 4 + q * 2 + 1] = __int_as_float(bi);
        }
        barrier();
        if (q == 0 && lane == 0 && store) {
            const float ov = xch[2 * XS + mine * 4 + 2];
            const int oi = __float_as_int(xch[2 * XS + mine * 4 + 3]);
            const bool take = (oi != 0x7fffffff) && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
            bi = take ? oi : bi;
            a.best[b] = bi == 0x7fffffff ? -1 : bi;
        }
    }
    // ---- pooled value heads (reference brokefish/nn/model.py:576-617) --------------------------------
    // The value row is the mean over the live tokens of the normalised stream ("pooled", mode 1) or
    // the final LayerNorm of the mean of the residual stream ("prenorm", mode 2); it goes through
    // the value rows of head tile 2 like a token, and the result is in White's frame, so it is
    // negated when Black is to move.
    if (a.vmode != 0) {
        float pv[NP][16], hv[NP][16];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const bool lv = (alive[p] >> t) & 1u;
            const float cdiv = (float)(__builtin_popcount(alive[p]) > 0 ? __builtin_popcount(alive[p]) : 1);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float v = lv ? (a.vmode == 1 ? hn[p][r] : x[p][r]) : 0.0f;
#pragma unroll
                for (int d = 16; d >= 1; d >>= 1) v = v + __shfl_xor(v, d);
                pv[p][r] = v / cdiv;
            }
        }
        if (a.vmode == 2) {
            layernorm2(pv, gp + C::G_NFG + 32 * tile, gp + C::G_NFB + 32 * tile, hv);
        } else {
#pragma unroll
            for (int p = 0; p < NP; p++)
#pragma unroll
                for (int r = 0; r < 16; r++) hv[p][r] = pv[p][r];
        }
        barrier();   // every wave has finished reading the normalised streams
#pragma unroll
        for (int p = 0; p < NP; p++) {
            float* const dst = reinterpret_cast<float*>(hid + p * C::HID_P);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = {hv[p][4 * j], hv[p][4 * j + 1], hv[p][4 * j + 2], hv[p][4 * j + 3]};
                *reinterpret_cast<v4f*>(dst + ((tile * 4 + j) * 64 + lane) * 4) = v;
            }
        }
        barrier();
        if (q == 2 && heads_here) {
            // head tile 2 once more, against the pooled row (every token column holds the same row);
            // its blocks are read straight from the stream, in the same order as above
            v16f hd = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            for (int f = 0; f < 8 * HB; f++) {
                const v4f w = *reinterpret_cast<const v4f*>(wsrc + (size_t)hseq0 * BLOCK + (size_t)f * FRAG);
                const v4f hvv = *reinterpret_cast<const v4f*>(hnb + (f * 64 + lane) * 4);
#pragma unroll
                for (int k = 0; k < 4; k++) hd = __builtin_amdgcn_mfma_f32_32x32x2f32(w[k], hvv[k], hd, 0, 0, 0);
            }
            if (lane == 32 && store) {
                const float v = value_of(hd);
                a.value[b] = ctrl_m > 0 ? v : -v;
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

template <bool TAPS, bool FP8 = false, bool PROF = false, int NPOS = 2>
hipError_t launch_duo(const KArgs& k, hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be requested once per kernel and device
    static std::atomic<unsigned long long> lds_set{0};
    constexpr int lds_bytes = Cfg<FP8, NPOS>::LDS_BYTES;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
    if (!(lds_set.load(std::memory_order_relaxed) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&duo_kernel<TAPS, FP8, PROF, NPOS>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) return e;
        lds_set.fetch_or(bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL((duo_kernel<TAPS, FP8, PROF, NPOS>), dim3((k.n + NPOS - 1) / NPOS), dim3(512), lds_bytes, stream, k);
    return hipGetLastError();
}

}  // namespace duo
}  // namespace bf
