// Single-launch quantised network evaluator for gfx950 (MI355X).
//
// One wavefront evaluates one position: the 32 tokens of a board are the 32 columns of
// every MFMA tile, and lanes l and l+32 share a token.  The residual stream
// (32 tokens x 256 channels, fp32) lives in registers in MFMA accumulator layout for all
// layers, so LayerNorm, the quantisers and the 32-token softmax are per-lane loops plus
// one exchange with lane ^ 32.  All weight GEMMs are computed transposed,
//     D[out_channel, token] = W[out_channel, k] * X^T[k, token]
// with v_mfma_i32_32x32x32_i8, so a requantised output tile is already a valid B operand
// of the next GEMM (the k order of an MFMA is free as long as both operands agree; the
// host packs the weights in that order).  int8 weight tiles stream from HBM/L2 through a
// double-buffered LDS ring with direct-to-LDS loads, 32 KiB per group, shared by the four
// boards of a workgroup.  Attention (QK^T, PV) and the heads run on v_mfma_f32_32x32x2f32,
// which accumulates as an exact chain of fused multiply-adds in k order.
//
// Arithmetic contract (what the CPU checker restates operation by operation):
//   embedding  ((sq + ts) + ct) + (clock + rep)                        fp32
//   LayerNorm  two partial sums per row (one per lane half), sequential over tiles then r
//   quantise   s = amax / qmax, q = rint(x / s)  (x / s as a correctly rounded quotient)
//   GEMM       exact int32; descale fl(fl(acc * sa) * sw) + b; several k-chunks are summed
//              in fp64 before the single cast to fp32
//   softmax    exp from bf_exp_neg, p * (1 / l)
// See include/brokefish_hip.h for the blob layouts.

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdio>
#include <cstring>

#include "brokefish_hip.h"

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

namespace bf {

constexpr int T = 32;
constexpr int THREADS = 256;
constexpr int WAVES = 4;
constexpr int FRAG = 1024;          // 64 lanes x 16 bytes
constexpr int BLOCK = 8 * FRAG;     // one output tile over a 256-wide k-chunk
constexpr int GROUP = 4 * BLOCK;    // unit of the LDS ring
constexpr int RING = 2 * GROUP;

constexpr int D = 256, F = 1024, NH = 8;
constexpr int NT = D / 32;          // tiles across the model width
constexpr int FT = F / 32;          // tiles across the FFN hidden width
constexpr int KCF = F / 256;        // k-chunks of the second FFN matmul
constexpr int LAYER_BLOCKS = 3 * NT + NT + FT + NT * KCF;
constexpr int LAYER_GROUPS = LAYER_BLOCKS / 4;
constexpr int HEAD_GROUPS = 3;
static_assert(LAYER_BLOCKS % 8 == 0, "ring slot of a block must not depend on the layer");

// per-layer side parameters, in floats
constexpr int O_LN1G = 0, O_LN1B = D, O_BQKV = 2 * D, O_BOUT = 5 * D, O_LN2G = 6 * D,
              O_LN2B = 7 * D, O_BFF1 = 8 * D, O_BFF2 = 8 * D + F, O_WSUM = 9 * D + F,
              O_SW = 9 * D + F + KCF * D;
constexpr int N_SW = 3 * D / 128 + D / 128 + F / 128 + D / 128;
constexpr int LAYER_FLOATS = O_SW + ((N_SW + 3) / 4) * 4;
constexpr int SW_QKV = 0, SW_OUT = 3 * D / 128, SW_FF1 = SW_OUT + D / 128, SW_FF2 = SW_FF1 + F / 128;
// global side parameters after the layers
constexpr int G_SQ = 0, G_TS = 64 * D, G_CT = G_TS + 12 * D, G_CLOCK = G_CT + 4 * D,
              G_REP = G_CLOCK + 101 * D, G_NFG = G_REP + 3 * D, G_NFB = G_NFG + D,
              GLOBAL_FLOATS = G_NFB + D;

struct KArgs {
    const uint16_t* boards;
    const int16_t* control;
    const uint8_t* rep;
    const uint64_t* mask;
    int n;
    const uint8_t* wstream;
    const float* fparams;
    void* policy;
    void* promo;
    float* value;
    int* best;
    int out_fp32, n_layers, l0, l1, n_value;
    float eps;
    bf_taps taps;
};

__device__ __forceinline__ constexpr int ch(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }

// value held by the other lane of this token (lane ^ 32)
__device__ __forceinline__ float partner(float v, int g) {
    const int iv = __float_as_int(v);
    const auto r = __builtin_amdgcn_permlane32_swap(iv, iv, false, false);
    return __int_as_float(g ? r[0] : r[1]);
}

// exp(x) for x <= 0; same operation sequence as the CPU checker's bfo_exp_neg
__device__ __forceinline__ float exp_neg(float x) {
    const float t = x * 1.44269504088896341f;
    const float n = __builtin_rintf(t);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    const float z = r * r;
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float y = __builtin_fmaf(p, z, r);
    y = y + 1.0f;
    const float s = __int_as_float(__float_as_int(y) + (((int)n) << 23));
    return (x >= -87.0f) ? s : 0.0f;
}

__device__ __forceinline__ float tanh_dev(float x) {
    const float a = __builtin_fabsf(x);
    const float e = exp_neg(-2.0f * a);
    float th = (1.0f - e) / (1.0f + e);
    th = (a > 9.0f) ? 1.0f : th;
    return __builtin_copysignf(th, x);
}

__device__ __forceinline__ v4f ldg4(const float* p) { return *reinterpret_cast<const v4f*>(p); }
__device__ __forceinline__ v4i ldg4i(const float* p) { return *reinterpret_cast<const v4i*>(p); }

extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];

// ---- LDS ring ----------------------------------------------------------------------

struct Stream {
    const uint8_t* base;  // wstream
    int pos;              // next position (in consumption order) to issue
    int body_groups;      // groups of the layers that run
    int first_gid;        // absolute group of position 0
    int head_gid;         // absolute group of the first head tile
    int total;            // positions in this launch
};

__device__ __forceinline__ void issue_group(Stream& st, int wave, int lane) {
    if (st.pos < st.total) {
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

// Called before the first block of every group: this group's bytes have landed, every
// wave is done with the previous group, so its half of the ring can be refilled.
__device__ __forceinline__ void ring_sync(Stream& st, int wave, int lane) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    issue_group(st, wave, lane);
}

#define BF_BLOCK(blk)                                  \
    ([&]() -> int {                                    \
        if (((blk) & 3) == 0) ring_sync(st, wave, lane); \
        return ((blk) & 7) * BLOCK;                    \
    }())

// acc[out_channel r][token] (weights as A) or acc[token r][out_channel] (SWAP, weights as B)
template <bool SWAP>
__device__ __forceinline__ v16i gemm_tile(int off, const v4i (&act)[8], int lane) {
    v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 8; s++) {
        const v4i w = *reinterpret_cast<const v4i*>(&ring[off + s * FRAG + lane * 16]);
        acc = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(act[s], w, acc, 0, 0, 0)
                   : __builtin_amdgcn_mfma_i32_32x32x32_i8(w, act[s], acc, 0, 0, 0);
    }
    return acc;
}

// ---- row operations -------------------------------------------------------------------

// signed int8 quantiser of one token row spread over two lanes; y is [tiles][16]
template <int NTILES>
__device__ __forceinline__ void quant_s8(const float (&y)[NTILES][16], int g, v4i (&q)[NTILES], float& sa) {
    float am = 0.0f;
#pragma unroll
    for (int n = 0; n < NTILES; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) am = __builtin_fmaxf(am, __builtin_fabsf(y[n][r]));
    am = __builtin_fmaxf(am, partner(am, g));
    sa = am > 0.0f ? am / 127.0f : 1.0f;
    const float inv = 1.0f / sa;
#pragma unroll
    for (int n = 0; n < NTILES; n++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned w = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float v = y[n][4 * j + i];
                // correctly rounded v / sa from the reciprocal and two fused corrections
                const float q0 = v * inv;
                const float rem = __builtin_fmaf(-q0, sa, v);
                const float qf = __builtin_fmaf(rem, inv, q0);
                // adding 1.5 * 2^23 rounds to nearest even and leaves the integer in the low bits
                const unsigned m = (unsigned)__float_as_int(qf + 12582912.0f);
                w |= (m & 0xffu) << (8 * i);
            }
            q[n][j] = (int)w;
        }
}

// LayerNorm of the residual rows, affine applied, in the fixed lane order
__device__ __forceinline__ void layernorm(const float (&x)[NT][16], const float* gamma, const float* beta,
                                          float eps, int g, float (&y)[NT][16]) {
    float s = 0.0f;
#pragma unroll
    for (int n = 0; n < NT; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) s = s + x[n][r];
    const float mean = (s + partner(s, g)) * (1.0f / D);
    float v = 0.0f;
#pragma unroll
    for (int n = 0; n < NT; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float d = x[n][r] - mean;
            v = __builtin_fmaf(d, d, v);
        }
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

template <bool TAPS>
__global__ __launch_bounds__(THREADS, 1) void eval_kernel(const KArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t = lane & 31, g = lane >> 5;
    const int board_raw = blockIdx.x * WAVES + wave;
    const bool valid = board_raw < a.n;
    const int b = valid ? board_raw : a.n - 1;  // idle waves shadow the last board, store nothing

    Stream st;
    st.base = a.wstream;
    st.pos = 0;
    st.body_groups = (a.l1 - a.l0) * LAYER_GROUPS;
    st.first_gid = a.l0 * LAYER_GROUPS;
    st.head_gid = a.n_layers * LAYER_GROUPS;
    st.total = st.body_groups + HEAD_GROUPS;
    issue_group(st, wave, lane);

    const float* gp = a.fparams + (size_t)a.n_layers * LAYER_FLOATS;

    // ---- embedding ---------------------------------------------------------------------
    float x[NT][16];
    const unsigned word = a.boards[(size_t)b * T + t];
    const int ctrl = a.control[b];
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
    const int nl_run = a.l1 - a.l0;
    for (int l = a.l0; l < a.l1; l++) {
        const float* lp = a.fparams + (size_t)l * LAYER_FLOATS;
        const size_t bl = (size_t)b * nl_run + (l - a.l0);  // tap row

        v4i xq[NT];
        float sa;
        {
            float y[NT][16];
            layernorm(x, lp + O_LN1G, lp + O_LN1B, a.eps, g, y);
            quant_s8<NT>(y, g, xq, sa);
        }
        if (TAPS && a.taps.qa_qkv && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(a.taps.qa_qkv + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = xq[n][j];
        }
        // activation scale of token ch(r, g), for the V tiles whose rows are tokens
        float sa_tok[16];
#pragma unroll
        for (int r = 0; r < 16; r++) sa_tok[r] = __shfl(sa, ch(r, g));

        // ---- attention, one head at a time ------------------------------------------------
        float o[NH][16];
#pragma unroll
        for (int h = 0; h < NH; h++) {
            float qf[16], kf[16], vf[16];
            {
                const v16i acc = gemm_tile<false>(BF_BLOCK(3 * h + 0), xq, lane);
                const float sw = lp[O_SW + SW_QKV + (32 * h) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f bi = ldg4(lp + O_BQKV + 32 * h + 8 * j + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        qf[4 * j + i] = ((float)acc[4 * j + i] * sa) * sw + bi[i];
                }
                if (TAPS && a.taps.acc_qkv && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_qkv[(bl * T + t) * 3 * D + 32 * h + ch(r, g)] = acc[r];
            }
            {
                const v16i acc = gemm_tile<false>(BF_BLOCK(3 * h + 1), xq, lane);
                const float sw = lp[O_SW + SW_QKV + (D + 32 * h) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f bi = ldg4(lp + O_BQKV + D + 32 * h + 8 * j + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        kf[4 * j + i] = ((float)acc[4 * j + i] * sa) * sw + bi[i];
                }
                if (TAPS && a.taps.acc_qkv && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_qkv[(bl * T + t) * 3 * D + D + 32 * h + ch(r, g)] = acc[r];
            }
            {
                // V tile transposed: lane = channel, registers = tokens
                const v16i acc = gemm_tile<true>(BF_BLOCK(3 * h + 2), xq, lane);
                const float sw = lp[O_SW + SW_QKV + (2 * D + 32 * h) / 128];
                const float bi = lp[O_BQKV + 2 * D + 32 * h + t];
#pragma unroll
                for (int r = 0; r < 16; r++) vf[r] = ((float)acc[r] * sa_tok[r]) * sw + bi;
                if (TAPS && a.taps.acc_qkv && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_qkv[(bl * T + ch(r, g)) * 3 * D + 2 * D + 32 * h + t] = acc[r];
            }
            // scores, transposed: lane = query token, register r = key ch(r, g)
            v16f sc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 16; r++) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[r], qf[r], sc, 0, 0, 0);
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
        }

        // ---- output projection + residual -------------------------------------------------
        {
            v4i oq[NT];
            float so;
            quant_s8<NT>(o, g, oq, so);
            if (TAPS && a.taps.qa_out && valid) {
#pragma unroll
                for (int n = 0; n < NT; n++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        *reinterpret_cast<int*>(a.taps.qa_out + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = oq[n][j];
            }
#pragma unroll
            for (int n = 0; n < NT; n++) {
                const v16i acc = gemm_tile<false>(BF_BLOCK(3 * NT + n), oq, lane);
                const float sw = lp[O_SW + SW_OUT + (32 * n) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f bi = ldg4(lp + O_BOUT + 32 * n + 8 * j + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        x[n][4 * j + i] = x[n][4 * j + i] + (((float)acc[4 * j + i] * so) * sw + bi[i]);
                }
                if (TAPS && a.taps.acc_out && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_out[(bl * T + t) * D + 32 * n + ch(r, g)] = acc[r];
            }
        }

        // ---- feed-forward ------------------------------------------------------------------
        {
            float y[NT][16];
            layernorm(x, lp + O_LN2G, lp + O_LN2B, a.eps, g, y);
            quant_s8<NT>(y, g, xq, sa);
        }
        if (TAPS && a.taps.qa_ff1 && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *reinterpret_cast<int*>(a.taps.qa_ff1 + (bl * T + t) * D + 32 * n + 8 * j + 4 * g) = xq[n][j];
        }
        v4i hq[KCF][8];
        float sh[KCF];
#pragma unroll
        for (int c = 0; c < KCF; c++) {
            float hf[8][16];
            float am = 0.0f;
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const int tile = 8 * c + s;
                const v16i acc = gemm_tile<false>(BF_BLOCK(4 * NT + tile), xq, lane);
                const float sw = lp[O_SW + SW_FF1 + (32 * tile) / 128];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f bi = ldg4(lp + O_BFF1 + 32 * tile + 8 * j + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = __builtin_fmaxf(((float)acc[4 * j + i] * sa) * sw + bi[i], 0.0f);
                        hf[s][4 * j + i] = v;
                        am = __builtin_fmaxf(am, v);
                    }
                }
                if (TAPS && a.taps.acc_ff1 && valid)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        a.taps.acc_ff1[(bl * T + t) * F + 32 * tile + ch(r, g)] = acc[r];
            }
            // unsigned quantiser over this 256-wide chunk; bytes stored as q - 128 for the
            // signed MFMA, the offset is added back through wsum
            am = __builtin_fmaxf(am, partner(am, g));
            const float s8 = am > 0.0f ? am / 255.0f : 1.0f;
            const float inv = 1.0f / s8;
            sh[c] = s8;
#pragma unroll
            for (int s = 0; s < 8; s++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    unsigned w = 0;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = hf[s][4 * j + i];
                        const float q0 = v * inv;
                        const float rem = __builtin_fmaf(-q0, s8, v);
                        const float qf = __builtin_fmaf(rem, inv, q0);
                        const unsigned m = (unsigned)__float_as_int(qf + 12582912.0f);
                        w |= (m & 0xffu) << (8 * i);
                    }
                    if (TAPS && a.taps.qa_ff2 && valid)
                        *reinterpret_cast<unsigned*>(a.taps.qa_ff2 + (bl * T + t) * F + 256 * c + 32 * s + 8 * j + 4 * g) = w;
                    hq[c][s][j] = (int)(w ^ 0x80808080u);
                }
        }
#pragma unroll
        for (int n = 0; n < NT; n++) {
            double o64[16];
#pragma unroll
            for (int c = 0; c < KCF; c++) {
                const v16i acc = gemm_tile<false>(BF_BLOCK(4 * NT + FT + n * KCF + c), hq[c], lane);
                const double sc = (double)sh[c];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4i ws = ldg4i(lp + O_WSUM + c * D + 32 * n + 8 * j + 4 * g);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int full = acc[4 * j + i] + ws[i];
                        // exact product, one rounding in the add: same as out += acc * sa in fp64
                        o64[4 * j + i] = c == 0 ? (double)full * sc
                                                : __builtin_fma((double)full, sc, o64[4 * j + i]);
                        if (TAPS && a.taps.acc_ff2 && valid)
                            a.taps.acc_ff2[((bl * KCF + c) * T + t) * D + 32 * n + 8 * j + 4 * g + i] = full;
                    }
                }
            }
            const float sw = lp[O_SW + SW_FF2 + (32 * n) / 128];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f bi = ldg4(lp + O_BFF2 + 32 * n + 8 * j + 4 * g);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    x[n][4 * j + i] = x[n][4 * j + i] + ((float)o64[4 * j + i] * sw + bi[i]);
            }
        }
        if (TAPS && a.taps.resid && valid) {
#pragma unroll
            for (int n = 0; n < NT; n++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    a.taps.resid[(bl * T + t) * D + 32 * n + ch(r, g)] = x[n][r];
        }
    }

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
        ring_sync(st, wave, lane);
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
}

}  // namespace bf

// ---- host side --------------------------------------------------------------------------------

static thread_local char g_err[512] = "";

static int fail(int code, const char* msg) {
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return code;
}

static bool shape_ok(const bf_shape* s) {
    return s && s->d_model == bf::D && s->d_ff == bf::F && s->n_heads == bf::NH && s->n_layers >= 1 &&
           (s->n_value == 1 || s->n_value == 3);
}

extern "C" size_t bf_wstream_bytes(const bf_shape* s) {
    if (!shape_ok(s)) return 0;
    return ((size_t)s->n_layers * bf::LAYER_GROUPS + bf::HEAD_GROUPS) * bf::GROUP;
}

extern "C" size_t bf_fparams_floats(const bf_shape* s) {
    if (!shape_ok(s)) return 0;
    return (size_t)s->n_layers * bf::LAYER_FLOATS + bf::GLOBAL_FLOATS;
}

extern "C" void bf_int8_q_max(double* s8, double* u8) {
    if (s8) *s8 = 127.0;
    if (u8) *u8 = 255.0;
}

extern "C" const char* bf_last_error(void) { return g_err; }

static int check_args(const bf_eval_args* a, bf::KArgs* k) {
    if (!a) return fail(BF_ERR_ARGUMENT, "args is NULL");
    if (!shape_ok(&a->shape))
        return fail(BF_ERR_UNSUPPORTED,
                    "unsupported network shape: this build carries d_model=256, n_heads=8, d_ff=1024, "
                    "n_layers>=1, n_value in {1,3}");
    if (a->n < 1 || a->n > (1ll << 28)) return fail(BF_ERR_ARGUMENT, "n must be in [1, 2^28]");
    if (!a->boards || !a->control || !a->rep) return fail(BF_ERR_ARGUMENT, "boards/control/rep must not be NULL");
    if (!a->wstream || !a->fparams) return fail(BF_ERR_ARGUMENT, "wstream/fparams must not be NULL");
    if (!a->policy || !a->promo || !a->value) return fail(BF_ERR_ARGUMENT, "policy/promo/value must not be NULL");
    if (((uintptr_t)a->wstream & 15) || ((uintptr_t)a->fparams & 15))
        return fail(BF_ERR_ARGUMENT, "wstream/fparams must be 16-byte aligned");
    if (((uintptr_t)a->policy & 15) || ((uintptr_t)a->promo & 7) || ((uintptr_t)a->boards & 1))
        return fail(BF_ERR_ARGUMENT, "policy must be 16-byte and promo 8-byte aligned");
    if (a->best_move && !a->mask) return fail(BF_ERR_ARGUMENT, "best_move needs a mask");
    memset(k, 0, sizeof(*k));
    k->boards = a->boards; k->control = a->control; k->rep = a->rep; k->mask = a->mask;
    k->n = (int)a->n;
    k->wstream = a->wstream; k->fparams = a->fparams;
    k->policy = a->policy; k->promo = a->promo; k->value = a->value; k->best = a->best_move;
    k->out_fp32 = a->out_fp32 ? 1 : 0;
    k->n_layers = a->shape.n_layers; k->n_value = a->shape.n_value; k->eps = a->shape.eps;
    k->l0 = 0; k->l1 = a->shape.n_layers;
    if (a->taps) {
        k->taps = *a->taps;
        if (a->taps->layer_begin || a->taps->layer_end) {
            k->l0 = a->taps->layer_begin; k->l1 = a->taps->layer_end;
            if (k->l0 < 0 || k->l1 > k->n_layers || k->l0 > k->l1)
                return fail(BF_ERR_ARGUMENT, "taps layer range must satisfy 0 <= begin <= end <= n_layers");
        }
        if (a->taps->x_in && ((uintptr_t)a->taps->x_in & 15)) return fail(BF_ERR_ARGUMENT, "x_in must be 16-byte aligned");
    }
    return BF_OK;
}

static int launch(const bf_eval_args* a, const bf::KArgs& k, hipStream_t stream) {
    const int grid = (k.n + bf::WAVES - 1) / bf::WAVES;
    if (a->taps)
        hipLaunchKernelGGL(bf::eval_kernel<true>, dim3(grid), dim3(bf::THREADS), bf::RING, stream, k);
    else
        hipLaunchKernelGGL(bf::eval_kernel<false>, dim3(grid), dim3(bf::THREADS), bf::RING, stream, k);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_err, sizeof(g_err), "kernel launch failed: %s", hipGetErrorString(e));
        return BF_ERR_LAUNCH;
    }
    return BF_OK;
}

extern "C" int bf_model_forward(const bf_eval_args* args, void* stream) {
    bf::KArgs k;
    const int rc = check_args(args, &k);
    if (rc) return rc;
    return launch(args, k, (hipStream_t)stream);
}

extern "C" double bf_time_kernel_ms(const bf_eval_args* args, void* stream, int warmup, int iters) {
    bf::KArgs k;
    int rc = check_args(args, &k);
    if (rc) return rc;
    if (iters < 1 || warmup < 0) return fail(BF_ERR_ARGUMENT, "iters must be >= 1 and warmup >= 0");
    hipStream_t s = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
        return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    for (int i = 0; i < warmup && !rc; i++) rc = launch(args, k, s);
    hipEventRecord(e0, s);
    for (int i = 0; i < iters && !rc; i++) rc = launch(args, k, s);
    hipEventRecord(e1, s);
    const hipError_t e = hipEventSynchronize(e1);
    float ms = 0.0f;
    hipEventElapsedTime(&ms, e0, e1);
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    if (rc) return rc;
    if (e != hipSuccess) return fail(BF_ERR_LAUNCH, hipGetErrorString(e));
    return (double)ms / iters;
}
