// Device code of the evaluator (see bf_args.h for the design notes).  Included by one
// translation unit per kernel variant so the variants compile in parallel.
#pragma once

#include <atomic>

#include "bf_device.hip.h"

namespace bf {

extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];   // ring, then two parameter buffers

// ---- LDS ring ----------------------------------------------------------------------

struct Stream {
    unsigned long long t_sync;  // cycles spent waiting in ring_sync (profile builds only)
    const uint8_t* base;  // wstream
    int pos;              // next position (in consumption order) to issue
    int body_groups;      // groups of the layers that run
    int first_gid;        // absolute group of position 0
    int head_gid;         // absolute group of the first head tile
    int total;            // positions in this launch
};

template <bool GUARDED>
__device__ __forceinline__ void issue_group(Stream& st, int wave, int lane) {
    // Inside the layers the next position always exists (the head tiles follow), so the
    // unguarded form keeps the layer body free of branches.
    if (!GUARDED || st.pos < st.total) {
        const int gid = st.pos < st.body_groups ? st.first_gid + st.pos
                                                : st.head_gid + (st.pos - st.body_groups);
        const uint8_t* src = st.base + (size_t)gid * GROUP + (size_t)wave * BLOCK + lane * 16;
        uint8_t* dst = ring + (st.pos & 1) * GROUP + wave * BLOCK;
#pragma unroll
        for (int s = 0; s < 8; s++)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(src + s * FRAG),
                (__attribute__((address_space(3))) void*)(dst + s * FRAG), 16, 0, 0);
    }
    st.pos++;
}

// One layer's side parameters (PARAM_BYTES) into parameter buffer `buf`.
__device__ __forceinline__ void issue_params(const float* fparams, int layer, int buf, int wave, int lane) {
    const uint8_t* src = reinterpret_cast<const uint8_t*>(fparams) + (size_t)layer * PARAM_BYTES + wave * FRAG + lane * 16;
    uint8_t* dst = ring + RING + buf * PARAM_BYTES + wave * FRAG;
#pragma unroll
    for (int i = 0; i < PARAM_BYTES / (WAVES * FRAG); i++)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(src + i * WAVES * FRAG),
            (__attribute__((address_space(3))) void*)(dst + i * WAVES * FRAG), 16, 0, 0);
}

// Called before the first block of a group is read from LDS: this group's bytes have
// landed, every wave has finished reading the previous group (its fragment reads have
// returned), so that half of the ring can be refilled.
template <bool GUARDED, bool PROF = false>
__device__ __forceinline__ void ring_sync(Stream& st, int wave, int lane) {
    unsigned long long t0 = 0;
    if (PROF) t0 = __builtin_readcyclecounter();
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (PROF) st.t_sync += __builtin_readcyclecounter() - t0;
    issue_group<GUARDED>(st, wave, lane);
}

// Fragments of block `blk` (index within the layer; LAYER_BLOCKS = block 0 of the next layer).
template <bool PROF>
__device__ __forceinline__ void load_frags(int blk, v4i (&fr)[8], Stream& st, int wave, int lane) {
    if ((blk & 3) == 0) ring_sync<false, PROF>(st, wave, lane);
    const int off = (blk & 7) * BLOCK;
#pragma unroll
    for (int s = 0; s < 8; s++) fr[s] = *reinterpret_cast<const v4i*>(&ring[off + s * FRAG + lane * 16]);
}

// LayerNorm of the residual rows, affine applied, in the fixed lane order; gamma/beta in LDS or global
__device__ __forceinline__ void layernorm(const float (&x)[NT][16], const float* gamma, const float* beta,
                                          float eps, int g, float (&y)[NT][16]) {
    // per lane: every tile's 16 values form one chain from zero, the two tile sums of a quarter of
    // the width are added, the four quarter sums are added in order; then the two lanes of the token
    static_assert(NT == 8, "two tiles per quarter of the width");
    float sg[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        float ts[2];
#pragma unroll
        for (int n = 0; n < 2; n++) {
            float s = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) s = s + x[2 * q + n][r];
            ts[n] = s;
        }
        sg[q] = ts[0] + ts[1];
    }
    const float s = ((sg[0] + sg[1]) + sg[2]) + sg[3];
    const float mean = (s + partner(s, g)) * (1.0f / D);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        float ts[2];
#pragma unroll
        for (int n = 0; n < 2; n++) {
            float v = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float d = x[2 * q + n][r] - mean;
                v = __builtin_fmaf(d, d, v);
            }
            ts[n] = v;
        }
        sg[q] = ts[0] + ts[1];
    }
    const float v = ((sg[0] + sg[1]) + sg[2]) + sg[3];
    const float var = (v + partner(v, g)) * (1.0f / D);
    const float rstd = 1.0f / __builtin_sqrtf(var + eps);
#pragma unroll
    for (int n = 0; n < NT; n++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v4f ga = ldg4(gamma + 32 * n + 8 * j + 4 * g);
            const v4f be = ldg4(beta + 32 * n + 8 * j + 4 * g);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float d = x[n][4 * j + i] - mean;
                y[n][4 * j + i] = __builtin_fmaf(d * rstd, ga[i], be[i]);
            }
        }
}

// ---- the kernel ------------------------------------------------------------------------

template <bool TAPS, bool PROF, bool FP8>
__global__ __launch_bounds__(THREADS, 1) void eval_kernel(const KArgs a) {
    typedef typename Acc<FP8>::type acc_t;
    unsigned long long ph[N_PHASES];
    unsigned long long t_mark = 0, t_begin = 0;
    if (PROF) {
#pragma unroll
        for (int i = 0; i < N_PHASES; i++) ph[i] = 0;
        t_mark = t_begin = __builtin_readcyclecounter();
    }
    // close the current phase: everything since the last mark is charged to `slot`
#define BF_PHASE(slot)                                              \
    do {                                                            \
        if (PROF) {                                                 \
            const unsigned long long now_ = __builtin_readcyclecounter(); \
            ph[slot] += now_ - t_mark;                              \
            t_mark = now_;                                          \
        }                                                           \
    } while (0)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = lane & 31, g = lane >> 5;
    const int board_raw = blockIdx.x * WAVES + wave;   // this wave's slot of the launch (also its workspace slot)
    // a skipped position keeps its wavefront (the workgroup's barriers need it) but stores nothing;
    // with a compacted leaf list slot j evaluates position leaf_index[j] while j < *leaf_count
    bool valid;
    int b;
    if (a.leaf_index) {
        valid = board_raw < a.n && board_raw < *a.leaf_count;
        b = __builtin_amdgcn_readfirstlane(a.leaf_index[valid ? board_raw : 0]);
        // an entry that is not a position of this launch is skipped like a slot past the count (the
        // wave stays for the workgroup's barriers and stores nothing); an idle wave may read an
        // unwritten entry
        valid = valid && b >= 0 && b < a.n;
        b = valid ? b : 0;
    } else {
        valid = board_raw < a.n && !(a.active && !a.active[board_raw < a.n ? board_raw : 0]);
        b = valid ? board_raw : a.n - 1;        // idle waves shadow the last board, store nothing
    }

    Stream st;
    st.t_sync = 0;
    st.base = a.wstream;
    st.pos = 0;
    st.body_groups = (a.l1 - a.l0) * LAYER_GROUPS;
    st.first_gid = a.l0 * LAYER_GROUPS;
    st.head_gid = a.n_layers * LAYER_GROUPS;
    st.total = st.body_groups + HEAD_GROUPS;
    issue_group<true>(st, wave, lane);
    if (a.l0 < a.l1) issue_params(a.fparams, a.l0, 0, wave, lane);

    const float* gp = a.fparams + (size_t)a.n_layers * PARAM_FLOATS;

    // ---- embedding ---------------------------------------------------------------------
    float x[NT][16];
    // An encoder-only launch (tap table with `alive`): the residual stream comes in through x_in, the
    // token mask through `alive`, the stream after the last layer goes out through resid_last, and
    // there are no board words and no heads.
    const bool enc_only = TAPS && a.taps.alive != nullptr;
    const unsigned word = enc_only ? (a.taps.alive[(size_t)b * T + t] ? 0u : 0x800u) : a.boards[(size_t)b * T + t];
    const int ctrl = enc_only ? 1 : a.control[b];
    const unsigned alive = (unsigned)__ballot(((word >> 11) & 1) == 0 && g == 0);
    if (TAPS && a.taps.x_in) {
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = ldg4(a.taps.x_in + ((size_t)b * T + t) * D + 32 * n + 8 * j + 4 * g);
#pragma unroll
                for (int i = 0; i < 4; i++) x[n][4 * j + i] = v[i];
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
        const float* e_sq = gp + G_SQ + (word & 63) * D + 4 * g;
        const float* e_ts = gp + G_TS + ts * D + 4 * g;
        const float* e_ct = gp + G_CT + ct * D + 4 * g;
        const float* e_ck = gp + G_CLOCK + clock * D + 4 * g;
        const float* e_rp = gp + G_REP + rp * D + 4 * g;
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = 32 * n + 8 * j;
                const v4f vs = ldg4(e_sq + c), vt = ldg4(e_ts + c), vc = ldg4(e_ct + c);
                const v4f vk = ldg4(e_ck + c), vr = ldg4(e_rp + c);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float per_board = vk[i] + vr[i];
                    float v = vs[i] + vt[i];
                    v = v + vc[i];
                    x[n][4 * j + i] = v + per_board;
                }
            }
    }
    if (TAPS && a.taps.embed && valid) {
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.embed[((size_t)b * T + t) * D + 32 * n + ch(r, g)] = x[n][r];
    }

    // ---- layers --------------------------------------------------------------------------
    // `fr` always holds the weight fragments of the next block to be multiplied: each
    // block's MFMA chain is followed at once by the LDS reads of the block after it.
    v4i fr[8];
    BF_PHASE(PH_EMBED);
    if (a.l0 < a.l1) load_frags<PROF>(0, fr, st, wave, lane);
    const int nl_run = a.l1 - a.l0;
    for (int l = a.l0; l < a.l1; l++) {
        const int li = l - a.l0;
        const float* lp = reinterpret_cast<const float*>(&ring[RING + (li & 1) * PARAM_BYTES]);
        const size_t bl = (size_t)b * nl_run + li;  // tap row
        const bool more = l + 1 < a.l1;
        // multiply by the block in `fr`, then fetch the fragments of the block after it
#define BF_MM(SWAP, blk, act)                                                   \
    ([&]() -> acc_t {                                                           \
        const acc_t r_ = mfma8<SWAP, FP8>(fr, act);                             \
        if ((blk) + 1 < LAYER_BLOCKS || more) load_frags<PROF>((blk) + 1, fr, st, wave, lane); \
        return r_;                                                              \
    }())

        v4i xq[NT];
        float sa;
        {
            float y[NT][16];
            layernorm(x, lp + O_LN1G, lp + O_LN1B, a.eps, g, y);
            quant_s8<NT, FP8>(y, g, xq, sa);
        }
        if (TAPS && a.taps.qa_qkv && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(a.taps.qa_qkv + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = xq[n][j];
        }
        BF_PHASE(PH_LN1);
        // activation scale of token ch(r, g), for the V tiles whose rows are tokens
        float sa_tok[16];
#pragma unroll
        for (int r = 0; r < 16; r++) sa_tok[r] = __shfl(sa, ch(r, g));

        // ---- attention, one head at a time, software-pipelined ---------------------------------
        // The three weight GEMMs of head h+1 are issued right after the score MFMAs of head h,
        // so the matrix pipe works through them while the vector ALU does head h's softmax, and
        // head h's PV MFMAs run under head h+1's epilogue.
        float o[NH][16];
        acc_t accq = BF_MM(false, 0, xq);
        acc_t acck = BF_MM(false, 1, xq);
        acc_t accv = BF_MM(true, 2, xq);   // V transposed: lane = channel, registers = tokens
#pragma unroll
        for (int h = 0; h < NH; h++) {
            float qf[16], kf[16], vf[16];
            {
                const float swq = lp[O_SW + SW_QKV + (32 * h) / 128];
                const float swk = lp[O_SW + SW_QKV + (D + 32 * h) / 128];
                const float swv = lp[O_SW + SW_QKV + (2 * D + 32 * h) / 128];
                const float bv = lp[O_BQKV + 2 * D + 32 * h + t];
                v4f bq[4], bk[4];
                load_tile16(lp + O_BQKV + 32 * h, g, bq);
                load_tile16(lp + O_BQKV + D + 32 * h, g, bk);
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        qf[4 * j + i] = (accf(accq, 4 * j + i) * sa) * swq + bq[j][i];
                        kf[4 * j + i] = (accf(acck, 4 * j + i) * sa) * swk + bk[j][i];
                    }
#pragma unroll
                for (int r = 0; r < 16; r++) vf[r] = (accf(accv, r) * sa_tok[r]) * swv + bv;
                if (TAPS && a.taps.acc_qkv && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        a.taps.acc_qkv[(bl * T + t) * 3 * D + 32 * h + ch(r, g)] = accbits(accq, r);
                        a.taps.acc_qkv[(bl * T + t) * 3 * D + D + 32 * h + ch(r, g)] = accbits(acck, r);
                        a.taps.acc_qkv[(bl * T + ch(r, g)) * 3 * D + 2 * D + 32 * h + t] = accbits(accv, r);
                    }
            }
            BF_PHASE(PH_QKV);
            // scores, transposed: lane = query token, register r = key ch(r, g)
            v16f sc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 16; r++) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[r], qf[r], sc, 0, 0, 0);
            if (h + 1 < NH) {
                accq = BF_MM(false, 3 * (h + 1) + 0, xq);
                acck = BF_MM(false, 3 * (h + 1) + 1, xq);
                accv = BF_MM(true, 3 * (h + 1) + 2, xq);
            }
            // The next layer's parameters can be fetched once every wave is inside this layer
            // (after the last layer the same layer is fetched again, into the idle buffer).
            if (h == 1) issue_params(a.fparams, more ? l + 1 : l, (li + 1) & 1, wave, lane);
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
            for (int r = 0; r < 16; r++) o[h][r] = oa[r];
            BF_PHASE(PH_ATTN);
        }

        // ---- output projection + residual -------------------------------------------------
        {
            v4i oq[NT];
            float so;
            quant_s8<NT, FP8>(o, g, oq, so);
            if (TAPS && a.taps.qa_out && valid) {
#pragma unroll
                for (int n = 0; n < NT; n++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        *reinterpret_cast<int*>(a.taps.qa_out + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = oq[n][j];
            }
            acc_t acc2[2];
            acc2[0] = BF_MM(false, 3 * NT, oq);
            v4f bcur[4];
            load_tile16(lp + O_BOUT, g, bcur);
#pragma unroll
            for (int n = 0; n < NT; n++) {
                if (n + 1 < NT) acc2[(n + 1) & 1] = BF_MM(false, 3 * NT + n + 1, oq);
                v4f bnxt[4];   // parameters are fetched one tile ahead of their use
                if (n + 1 < NT) load_tile16(lp + O_BOUT + 32 * (n + 1), g, bnxt);
                const acc_t acc = acc2[n & 1];
                const float sw = lp[O_SW + SW_OUT + (32 * n) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        x[n][4 * j + i] = x[n][4 * j + i] + ((accf(acc, 4 * j + i) * so) * sw + bcur[j][i]);
                pin16(x[n]);
                // This tile of the residual stream is final until the FFN's last epilogue:
                // copy it to the workspace now (one coalesced 1 KiB store per register quad),
                // tile by tile, so the copies do not arrive at the memory system as one burst.
                // The registers stay live through LayerNorm 2 and are released after it.
                {
                    float* xp = a.xpark + (size_t)board_raw * (T * D) + lane * 4;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const v4f v = {x[n][4 * j], x[n][4 * j + 1], x[n][4 * j + 2], x[n][4 * j + 3]};
                        *reinterpret_cast<v4f*>(xp + (n * 4 + j) * 256) = v;
                    }
                }
                if (TAPS && a.taps.acc_out && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_out[(bl * T + t) * D + 32 * n + ch(r, g)] = accbits(acc, r);
#pragma unroll
                for (int j = 0; j < 4; j++) bcur[j] = bnxt[j];
            }
        }

        BF_PHASE(PH_OUT);
        // ---- feed-forward ------------------------------------------------------------------
        {
            float y[NT][16];
            layernorm(x, lp + O_LN2G, lp + O_LN2B, a.eps, g, y);
            quant_s8<NT, FP8>(y, g, xq, sa);
        }
        BF_PHASE(PH_LN2);
        if (TAPS && a.taps.qa_ff1 && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(a.taps.qa_ff1 + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = xq[n][j];
        }
        v4i hq[KCF][8];
        float sh[KCF];
        {
            acc_t acc2[2];
            acc2[0] = BF_MM(false, 4 * NT, xq);
            float hf[8][16];
            float am = 0.0f;
            v4f bcur[4];
            load_tile16(lp + O_BFF1, g, bcur);
#pragma unroll
            for (int tile = 0; tile < FT; tile++) {
                const int c = tile / 8, s = tile % 8;
                if (tile + 1 < FT) acc2[(tile + 1) & 1] = BF_MM(false, 4 * NT + tile + 1, xq);
                v4f bnxt[4];
                if (tile + 1 < FT) load_tile16(lp + O_BFF1 + 32 * (tile + 1), g, bnxt);
                const acc_t acc = acc2[tile & 1];
                const float sw = lp[O_SW + SW_FF1 + (32 * tile) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = __builtin_fmaxf((accf(acc, 4 * j + i) * sa) * sw + bcur[j][i], 0.0f);
                        hf[s][4 * j + i] = v;
                        am = __builtin_fmaxf(am, v);
                    }
                pin16(hf[s]);
#pragma unroll
                for (int j = 0; j < 4; j++) bcur[j] = bnxt[j];
                if (TAPS && a.taps.acc_ff1 && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_ff1[(bl * T + t) * F + 32 * tile + ch(r, g)] = accbits(acc, r);
                if (s == 7) {
                    // int8: unsigned quantiser over this 256-wide chunk; bytes stored as q - 128
                    // for the signed MFMA, the offset is added back through wsum.
                    // e4m3: the ordinary signed quantiser (the values are non-negative).
                    am = __builtin_fmaxf(am, partner(am, g));
                    const float s8 = am > 0.0f ? am / (FP8 ? 8.0f : 255.0f) : 1.0f;
                    const float inv = 1.0f / s8;
                    sh[c] = s8;
#pragma unroll
                    for (int s2 = 0; s2 < 8; s2++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const unsigned w = quant4<FP8>(hf[s2][4 * j], hf[s2][4 * j + 1], hf[s2][4 * j + 2],
                                                           hf[s2][4 * j + 3], s8, inv);
                            if (TAPS && a.taps.qa_ff2 && valid)
                                *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl * T + t) * F + 256 * c + 32 * s2 + 8 * j + 4 * g) = w;
                            hq[c][s2][j] = (int)(FP8 ? w : (w ^ 0x80808080u));
                        }
                    am = 0.0f;
                }
            }
        }
        BF_PHASE(PH_FF1);
        {
            acc_t acc2[2];
            acc2[0] = BF_MM(false, 4 * NT + FT, hq[0]);
            double o64[16];   // int8: float64 sum over the k-chunks, as the reference's emulation
            float o32[16];    // e4m3: fp32 sum over the k-tiles
            v4i wcur[4];
            if (!FP8) load_tile16i(lp + O_WSUM, g, wcur);
            v4f bout[4];
#pragma unroll
            for (int idx = 0; idx < NT * KCF; idx++) {
                const int n = idx / KCF, c = idx % KCF;
                if (idx + 1 < NT * KCF) acc2[(idx + 1) & 1] = BF_MM(false, 4 * NT + FT + idx + 1, hq[(idx + 1) % KCF]);
                v4i wnxt[4];
                if (!FP8 && idx + 1 < NT * KCF)
                    load_tile16i(lp + O_WSUM + ((idx + 1) % KCF) * D + 32 * ((idx + 1) / KCF), g, wnxt);
                if (c == 0) {
                    load_tile16(lp + O_BFF2 + 32 * n, g, bout);   // used three blocks later
                    // bring this tile of the parked residual stream back, three blocks ahead
                    const float* xp = a.xpark + (size_t)board_raw * (T * D) + lane * 4;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const v4f v = *reinterpret_cast<const v4f*>(xp + (n * 4 + j) * 256);
#pragma unroll
                        for (int i = 0; i < 4; i++) x[n][4 * j + i] = v[i];
                    }
                }
                const acc_t acc = acc2[idx & 1];
                // weight scale of this (128-row block, k-chunk); int8 packs the same value for every chunk
                const float sw = lp[O_SW + SW_FF2 + ((32 * n) / 128) * KCF + c];
                if constexpr (FP8) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float part = (accf(acc, i) * sh[c]) * sw;
                        o32[i] = c == 0 ? part : o32[i] + part;
                        if (TAPS && a.taps.acc_ff2 && valid)
                            a.taps.acc_ff2[((bl * KCF + c) * T + t) * D + 32 * n + ch(i, g)] = accbits(acc, i);
                    }
                } else {
                    const double sc = (double)sh[c];
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int full = accbits(acc, 4 * j + i) + wcur[j][i];
                            // exact product, one rounding in the add: same as out += acc * sa in fp64
                            o64[4 * j + i] = c == 0 ? (double)full * sc
                                                    : __builtin_fma((double)full, sc, o64[4 * j + i]);
                            if (TAPS && a.taps.acc_ff2 && valid)
                                a.taps.acc_ff2[((bl * KCF + c) * T + t) * D + 32 * n + 8 * j + 4 * g + i] = full;
                        }
                }
                if (c == KCF - 1) {
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            float upd;
                            if constexpr (FP8) upd = o32[4 * j + i] + bout[j][i];
                            else upd = (float)o64[4 * j + i] * sw + bout[j][i];
                            x[n][4 * j + i] = x[n][4 * j + i] + upd;
                        }
                    pin16(x[n]);
                } else if constexpr (FP8) {
                    pin16(o32);
                } else {
#pragma unroll
                    for (int i = 0; i < 16; i++) pin(o64[i]);
                }
                if (!FP8) {
#pragma unroll
                    for (int j = 0; j < 4; j++) wcur[j] = wnxt[j];
                }
            }
        }
#undef BF_MM
        BF_PHASE(PH_FF2);
        if (TAPS && a.taps.resid && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    a.taps.resid[(bl * T + t) * D + 32 * n + ch(r, g)] = x[n][r];
        }
    }
    if (TAPS && a.taps.resid_last && valid) {
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.resid_last[((size_t)b * T + t) * D + 32 * n + ch(r, g)] = x[n][r];
    }
    if (enc_only) return;   // the same for every wave of the launch

    // ---- final norm and heads ------------------------------------------------------------------
    float hn[NT][16];
    layernorm(x, gp + G_NFG, gp + G_NFB, a.eps, g, hn);
    if (TAPS && a.taps.normed && valid) {
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                a.taps.normed[((size_t)b * T + t) * D + 32 * n + ch(r, g)] = hn[n][r];
    }
    v16f head[3];
#pragma unroll
    for (int m = 0; m < 3; m++) {
        // one 32 KiB group per head tile
        ring_sync<true, PROF>(st, wave, lane);
        const int off = (m & 1) * GROUP;
        v16f acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int n = 0; n < NT; n++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f w = *reinterpret_cast<const v4f*>(&ring[off + (n * 4 + j) * FRAG + lane * 16]);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w[i], hn[n][4 * j + i], acc, 0, 0, 0);
            }
        head[m] = acc;
    }
    BF_PHASE(PH_HEADS);
    // Nothing may leave before every wave has finished with the ring (no further sync follows).
    if (!valid) return;

    // value: king token of the side to move, lane half 1 holds head rows 68..70 in registers 0..2
    const int king = ctrl < 0 ? 31 : 15;
    if (lane == 32 + king) {
        float v;
        if (a.n_value == 1) {
            v = tanh_dev(head[2][0]);
        } else {
            const float r0 = head[2][0], r1 = head[2][1], r2 = head[2][2];
            const float mx = __builtin_fmaxf(__builtin_fmaxf(r0, r1), r2);
            const float e0 = exp_neg(r0 - mx), e1 = exp_neg(r1 - mx), e2 = exp_neg(r2 - mx);
            v = (e2 - e0) / ((e0 + e1) + e2);
        }
        a.value[b] = v;
    }
    // promo: head rows 64..67 are registers 0..3 of lane half 0
    if (g == 0) {
        if (a.out_fp32) {
            const v4f v = {head[2][0], head[2][1], head[2][2], head[2][3]};
            *reinterpret_cast<v4f*>((float*)a.promo + ((size_t)b * T + t) * 4) = v;
        } else {
            const v4h v = {(_Float16)head[2][0], (_Float16)head[2][1], (_Float16)head[2][2], (_Float16)head[2][3]};
            *reinterpret_cast<v4h*>((_Float16*)a.promo + ((size_t)b * T + t) * 4) = v;
        }
    }
    // policy, with the optional legal-move AND and argmax
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    unsigned long long mw = ~0ull;
    if (a.mask) mw = a.mask[(size_t)b * T + t];
#pragma unroll
    for (int m = 0; m < 2; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int sq = 32 * m + 8 * j + 4 * g + i;
                const bool legal = (mw >> sq) & 1ull;
                v[i] = legal ? head[m][4 * j + i] : -__builtin_inff();
                // squares are visited in increasing order within a lane, so '>' keeps the lowest
                if (legal && (bi == 0x7fffffff || v[i] > bv)) { bv = v[i]; bi = t * 64 + sq; }
            }
            const size_t at = ((size_t)b * T + t) * 64 + 32 * m + 8 * j + 4 * g;
            if (a.out_fp32) {
                const v4f vv = {v[0], v[1], v[2], v[3]};
                *reinterpret_cast<v4f*>((float*)a.policy + at) = vv;
            } else {
                const v4h vv = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                *reinterpret_cast<v4h*>((_Float16*)a.policy + at) = vv;
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
        if (lane == 0) a.best[b] = bi == 0x7fffffff ? -1 : bi;
    }
    if (PROF) {
        BF_PHASE(PH_STORE);
        ph[PH_SYNC] = st.t_sync;
        ph[PH_TOTAL] = __builtin_readcyclecounter() - t_begin;
        if (lane == 0 && a.profile)
#pragma unroll
            for (int i = 0; i < N_PHASES; i++) atomicAdd(&a.profile[i], ph[i]);
    }
#undef BF_PHASE
}


template <bool TAPS, bool PROF, bool FP8>
hipError_t launch_variant(const KArgs& k, int grid, hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be requested once per kernel and device (one bit
    // per device ordinal; a device beyond the mask asks every time)
    static std::atomic<unsigned long long> lds_set{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
    if (!(lds_set.load(std::memory_order_relaxed) & bit)) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&eval_kernel<TAPS, PROF, FP8>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) return e;
        lds_set.fetch_or(bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL((eval_kernel<TAPS, PROF, FP8>), dim3(grid), dim3(THREADS), LDS_BYTES, stream, k);
    return hipGetLastError();
}

}  // namespace bf