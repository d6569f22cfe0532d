// Edge expansion behind the evaluator: logits + legal-move words -> the edges of a search node.
//
// For every position: enumerate the set bits of the 32 legal-move words in canonical order
// (ascending slot, then square; a pawn move onto the last rank fans out into four edges in the
// order N B R Q), give each edge the unnormalised log-prior
//     policy[slot][square]  (+ log_softmax(promo[slot])[type] for a promotion edge),
// keep the E largest if there are more than E (ties by canonical order, survivors stay in
// canonical order), softmax over the survivors, and write move codes, fp16 priors, the edge
// count, the mass dropped by the truncation and the value mapped from [-1,1] to [0,1].
// Restates reference docs/reference/search.md:616-636 and brokefish/search/torch_impl.py:962-1033.
//
// One wavefront per position: lane l owns half a mask word (slot l/2, squares 32*(l%2) ..+31), so
// lane order is canonical order and an edge's index is a prefix sum over lanes.  A position has
// some 30 legal moves over its 64 half-words, so the lanes first lay the candidates out in LDS
// in canonical order (a lane walks only the set bits of its half-word, its logits staged in LDS)
// and then take one to four candidates each: softmax, truncation and the stores are lane-parallel
// over candidates, counts and ranks come from ballots.  The truncation threshold (the E-th largest
// log-prior) is found by bisection on the ordered bit pattern of the float.  A mask with more
// candidates than the layout holds (256; no legal position has them) is handled without it, every
// pass walking the lanes' set bits again.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdint>
#include <cstdio>

#include "bf_args.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int PAWN = 0;          // reference docs/reference/spec.md:47
constexpr int PROMO_SHIFT = 11;  // brokefish/search/torch_impl.py:61-62

struct KExpand {
    const void* policy;
    const void* promo;
    const float* value;
    const uint64_t* mask;
    const uint16_t* boards;
    const int16_t* control;
    const uint8_t* active;
    const int* leaf_index;        // optional compacted list: slot j expands position leaf_index[j] for j < *leaf_count
    const int* leaf_count;
    int n, E, logits_fp32;
    int16_t* edge_move;
    _Float16* edge_prior;
    int* n_edges;
    int* count;
    float* dropped;
    _Float16* node_value;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}
__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
    return v;
}
// exclusive prefix sum over the 64 lanes
__device__ __forceinline__ int wave_exclusive(int v, int lane) {
    int inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(inc, d);
        if (lane >= d) inc += o;
    }
    return inc - v;
}
// bit pattern whose unsigned order is the order of the floats
__device__ __forceinline__ unsigned ordered(float f) {
    const unsigned u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// lanes below this one whose bit is set in a ballot
__device__ __forceinline__ int lanes_below(unsigned long long ballot) {
    return __builtin_amdgcn_mbcnt_hi((unsigned)(ballot >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)ballot, 0));
}
// what one lane of this wave wrote to LDS is read by another: LDS operations of a wave are carried
// out in program order, the fences keep the compiler from changing that order
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int EXPAND_WAVES = 4;       // positions per workgroup
constexpr int CAND_CAP = 256;         // candidates a wave lays out in LDS (no legal chess position has more)

// FP32: the logits come as float32 (parity runs) instead of fp16 (the search contract); the staged
// rows are then twice as large, which costs resident wavefronts, so the two are separate kernels.
template <bool FP32>
__global__ __launch_bounds__(64 * EXPAND_WAVES) void expand_kernel(const KExpand a) {
    constexpr int ROW_STRIDE = (FP32 ? 128 : 64) + 16;   // bytes per lane of staged logits + a pad that spreads the banks
    __shared__ __attribute__((aligned(16))) char row_lds[EXPAND_WAVES][64 * ROW_STRIDE];
    __shared__ float cand_l[EXPAND_WAVES][CAND_CAP];
    __shared__ int16_t cand_c[EXPAND_WAVES][CAND_CAP];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int b = blockIdx.x * EXPAND_WAVES + wv;
    if (b >= a.n) return;                       // no workgroup barrier below: a wave may leave
    if (a.leaf_index) {
        if (b >= *a.leaf_count) return;
        b = __builtin_amdgcn_readfirstlane(a.leaf_index[b]);
        if ((unsigned)b >= (unsigned)a.n) return;   // not a position of this launch
    }
    if (a.active && !a.active[b]) return;
    const int p = lane >> 1, half = lane & 1;

    const unsigned word = a.boards[(size_t)b * 32 + p];
    const int ctrl = a.control[b];
    const bool pawn = ((word >> 11) & 1u) == 0 && ((word >> 6) & 7u) == PAWN;
    const uint64_t m64 = a.mask[(size_t)b * 32 + p];
    const unsigned mh = half ? (unsigned)(m64 >> 32) : (unsigned)m64;
    // last rank of the side to move: rank 7 (squares 56..63) for white, rank 0 for black
    const unsigned last = ctrl < 0 ? (half == 0 ? 0xFFu : 0u) : (half == 1 ? 0xFF000000u : 0u);
    const unsigned pr = pawn ? (mh & last) : 0u;

    const int cnt = __popc(mh) + 3 * __popc(pr);
    const int before = wave_exclusive(cnt, lane);
    const int total = __shfl(before + cnt, 63);

    // A lane that has moves stages its 32 policy logits in LDS, where the walks below pick the
    // ones its mask names (a lane without a move, which is most of them, loads nothing).
    char* const myrow = row_lds[wv] + lane * ROW_STRIDE;
    if (mh) {
        if constexpr (FP32) {
            const float* row = (const float*)a.policy + ((size_t)b * 32 + p) * 64 + 32 * half;
#pragma unroll
            for (int j = 0; j < 8; j++) *reinterpret_cast<v4f*>(myrow + 16 * j) = *reinterpret_cast<const v4f*>(row + 4 * j);
        } else {
            const _Float16* row = (const _Float16*)a.policy + ((size_t)b * 32 + p) * 64 + 32 * half;
#pragma unroll
            for (int j = 0; j < 4; j++) *reinterpret_cast<v8h*>(myrow + 16 * j) = *reinterpret_cast<const v8h*>(row + 8 * j);
        }
    }
    // its slot's promotion log-probabilities, where a pawn reaches the last rank
    float lp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (pr) {
        float x[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            x[k] = FP32 ? ((const float*)a.promo)[((size_t)b * 32 + p) * 4 + k]
                        : (float)((const _Float16*)a.promo)[((size_t)b * 32 + p) * 4 + k];
        const float mx = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        const float s = ((__expf(x[0] - mx) + __expf(x[1] - mx)) + __expf(x[2] - mx)) + __expf(x[3] - mx);
        const float ls = __logf(s);
#pragma unroll
        for (int k = 0; k < 4; k++) lp[k] = (x[k] - mx) - ls;
    }
    // visit this lane's candidates in canonical order: f(log-prior, move code)
    auto each = [&](auto&& f) {
        unsigned m = mh;
        while (m) {
            const int i = __builtin_ctz(m);
            m &= m - 1;
            const float l = FP32 ? reinterpret_cast<const float*>(myrow)[i] : (float)reinterpret_cast<const _Float16*>(myrow)[i];
            const int mv = p * 64 + 32 * half + i;
            if ((pr >> i) & 1u) {
#pragma unroll
                for (int k = 0; k < 4; k++) f(l + lp[k], mv | (k << PROMO_SHIFT));
            } else {
                f(l, mv);
            }
        }
    };
    int16_t* const em = a.edge_move + (size_t)b * a.E;
    _Float16* const ep = a.edge_prior + (size_t)b * a.E;
    const bool trunc = total > a.E;
    int n_edges;
    float s_all, s_keep;

    if (total <= CAND_CAP) {
        // ---- the candidates laid out in LDS in canonical order, then one to four per lane ----------
        float* const cl = cand_l[wv];
        int16_t* const cc = cand_c[wv];
        {
            int j = before;
            each([&](float l, int code) {
                cl[j] = l;
                cc[j] = (int16_t)code;
                j++;
            });
        }
        wave_lds_sync();
        constexpr int R = CAND_CAP / 64;
        float l[R], e[R];
        int code[R];
        bool has[R];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int idx = lane + 64 * r;
            has[r] = idx < total;
            l[r] = has[r] ? cl[idx] : -INFINITY;
            code[r] = has[r] ? cc[idx] : 0;
            mx = fmaxf(mx, l[r]);
        }
        mx = wave_max(mx);
        float sa = 0.0f;
#pragma unroll
        for (int r = 0; r < R; r++) {
            e[r] = has[r] ? __expf(l[r] - mx) : 0.0f;
            sa += e[r];
        }
        s_all = wave_sum(sa);
        if (!trunc) {
            // everything survives, in place
            n_edges = total;
            s_keep = s_all;
            const float inv = 1.0f / s_keep;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (has[r]) {
                    em[lane + 64 * r] = (int16_t)code[r];
                    ep[lane + 64 * r] = (_Float16)(e[r] * inv);
                }
        } else {
            // T = ordered pattern of the E-th largest log-prior, `need` ties at T survive
            unsigned o[R];
#pragma unroll
            for (int r = 0; r < R; r++) o[r] = has[r] ? ordered(l[r]) : 0u;
            unsigned T = 0;
#pragma clang loop unroll(disable)
            for (int bit = 31; bit >= 0; bit--) {
                const unsigned cand = T | (1u << bit);
                int c = 0;
#pragma unroll
                for (int r = 0; r < R; r++) c += __popcll(__ballot(has[r] && o[r] >= cand));
                if (c >= a.E) T = cand;
            }
            int gt = 0;
#pragma unroll
            for (int r = 0; r < R; r++) gt += __popcll(__ballot(has[r] && o[r] > T));
            const int need = a.E - gt;
            int ties = 0, kept_before = 0;
            float sk = 0.0f;
            bool keep[R];
            int pos[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const bool eq = has[r] && o[r] == T;
                const unsigned long long eqb = __ballot(eq);
                keep[r] = has[r] && (o[r] > T || (eq && ties + lanes_below(eqb) < need));
                ties += __popcll(eqb);
                const unsigned long long kb = __ballot(keep[r]);
                pos[r] = kept_before + lanes_below(kb);
                kept_before += __popcll(kb);
                sk += keep[r] ? e[r] : 0.0f;
            }
            n_edges = kept_before;
            s_keep = wave_sum(sk);
            const float inv = 1.0f / s_keep;
#pragma unroll
            for (int r = 0; r < R; r++)
                if (keep[r]) {
                    em[pos[r]] = (int16_t)code[r];
                    ep[pos[r]] = (_Float16)(e[r] * inv);
                }
        }
    } else {
        // ---- more candidates than the layout holds (no legal position: an arbitrary mask): nothing
        // is stored per candidate, every pass walks the lane's squares again ---------------------------
        float mx = -INFINITY;
        each([&](float l, int) { mx = fmaxf(mx, l); });
        mx = wave_max(mx);
        unsigned T = 0;
        int need = 0, tie_before = 0;
        if (trunc) {
#pragma clang loop unroll(disable)
            for (int bit = 31; bit >= 0; bit--) {
                const unsigned cand = T | (1u << bit);
                int c = 0;
                each([&](float l, int) { c += ordered(l) >= cand; });
                if (wave_sum(c) >= a.E) T = cand;
            }
            int gt = 0, eq = 0;
            each([&](float l, int) {
                const unsigned o = ordered(l);
                gt += o > T;
                eq += o == T;
            });
            need = a.E - wave_sum(gt);
            tie_before = wave_exclusive(eq, lane);
        }
        // one pass: kept count of this lane, softmax denominators over all and over the survivors
        int kept = 0, tie = tie_before;
        float sa = 0.0f, sk = 0.0f;
        each([&](float l, int) {
            const float e = __expf(l - mx);
            sa += e;
            bool keep = true;
            if (trunc) {
                const unsigned o = ordered(l);
                keep = o > T || (o == T && tie < need);
                tie += o == T;
            }
            if (keep) { kept++; sk += e; }
        });
        s_all = wave_sum(sa);
        s_keep = wave_sum(sk);
        int pos = wave_exclusive(kept, lane);
        n_edges = __shfl(pos + kept, 63);
        // write the survivors in canonical order
        const float inv = 1.0f / s_keep;
        tie = tie_before;
        each([&](float l, int code) {
            bool keep = true;
            if (trunc) {
                const unsigned o = ordered(l);
                keep = o > T || (o == T && tie < need);
                tie += o == T;
            }
            if (keep) {
                em[pos] = (int16_t)code;
                ep[pos] = (_Float16)(__expf(l - mx) * inv);
                pos++;
            }
        });
    }
    // unused edge slots read as no edge
    for (int i = n_edges + lane; i < a.E; i += 64) {
        em[i] = 0;
        ep[i] = (_Float16)0.0f;
    }
    if (lane == 0) {
        a.n_edges[b] = n_edges;
        if (a.count) a.count[b] = total;
        if (a.dropped) a.dropped[b] = trunc ? (s_all - s_keep) / s_all : 0.0f;
        if (a.node_value) a.node_value[b] = (_Float16)((a.value[b] + 1.0f) / 2.0f);
    }
}

}  // namespace

// Order-preserving compaction of the leaf flags by one workgroup of 1024 lanes: per pass each lane
// takes one flag; a wave's ballot gives the rank inside the wave, the 16 wave totals are scanned
// through LDS, and the running total carries over the passes.
__global__ __launch_bounds__(1024) void compact_kernel(const uint8_t* flags, int n, int* leaf_index, int* leaf_count) {
    __shared__ int wave_total[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int base = 0;
    for (int lo = 0; lo < n; lo += 1024) {
        const int i = lo + (int)threadIdx.x;
        const bool on = i < n && flags[i] != 0;
        const unsigned long long vote = __ballot(on);
        const int rank = __builtin_popcountll(vote & ((1ull << lane) - 1ull));
        if (lane == 0) wave_total[wave] = __builtin_popcountll(vote);
        __syncthreads();
        int before = 0, all = 0;
        for (int w = 0; w < 16; w++) {
            const int c = wave_total[w];
            before += w < wave ? c : 0;
            all += c;
        }
        if (on) leaf_index[base + before + rank] = i;
        base += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) *leaf_count = base;
}

extern "C" int bf_compact_leaves(const uint8_t* flags, int64_t n, int32_t* leaf_index, int32_t* leaf_count, void* stream) {
    auto fail = [](int code, const char* msg) {
        bf::set_error(msg);
        return code;
    };
    if (!flags || !leaf_index || !leaf_count) return fail(BF_ERR_ARGUMENT, "flags/leaf_index/leaf_count must not be NULL");
    if (n < 1 || n > (1ll << 28)) return fail(BF_ERR_ARGUMENT, "n must be in [1, 2^28]");
    if (((uintptr_t)leaf_index & 3) || ((uintptr_t)leaf_count & 3)) return fail(BF_ERR_ARGUMENT, "leaf_index / leaf_count must be 4-byte aligned");
    hipLaunchKernelGGL(compact_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, flags, (int)n, leaf_index, leaf_count);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[256];
        snprintf(msg, sizeof(msg), "kernel launch failed: %s", hipGetErrorString(e));
        return fail(BF_ERR_LAUNCH, msg);
    }
    return BF_OK;
}

extern "C" int bf_expand(const bf_expand_args* a, void* stream) {
    auto fail = [](int code, const char* msg) {
        bf::set_error(msg);
        return code;
    };
    if (!a) return fail(BF_ERR_ARGUMENT, "args is NULL");
    if (a->n < 1 || a->n > (1ll << 28)) return fail(BF_ERR_ARGUMENT, "n must be in [1, 2^28]");
    if (a->max_edges < 1 || a->max_edges > 255) return fail(BF_ERR_ARGUMENT, "max_edges must be in [1, 255]");
    if (!a->policy || !a->promo || !a->mask || !a->boards || !a->control)
        return fail(BF_ERR_ARGUMENT, "policy/promo/mask/boards/control must not be NULL");
    if (!a->edge_move || !a->edge_prior || !a->n_edges) return fail(BF_ERR_ARGUMENT, "edge_move/edge_prior/n_edges must not be NULL");
    if (a->node_value && !a->value) return fail(BF_ERR_ARGUMENT, "node_value needs value");
    if (((uintptr_t)a->policy & 15) || ((uintptr_t)a->mask & 7) || ((uintptr_t)a->promo & 1))
        return fail(BF_ERR_ARGUMENT, "policy must be 16-byte and mask 8-byte aligned");
    KExpand k;
    k.policy = a->policy; k.promo = a->promo; k.value = a->value; k.mask = a->mask;
    if ((a->leaf_index == nullptr) != (a->leaf_count == nullptr)) return fail(BF_ERR_ARGUMENT, "leaf_index and leaf_count come together");
    if (a->leaf_index && a->active) return fail(BF_ERR_ARGUMENT, "a compacted leaf list replaces the active flags: pass one of them");
    k.boards = a->boards; k.control = a->control; k.active = a->active;
    k.leaf_index = a->leaf_index; k.leaf_count = a->leaf_count;
    k.n = (int)a->n; k.E = a->max_edges; k.logits_fp32 = a->logits_fp32 ? 1 : 0;
    k.edge_move = a->edge_move; k.edge_prior = reinterpret_cast<_Float16*>(a->edge_prior);
    k.n_edges = a->n_edges; k.count = a->count; k.dropped = a->dropped;
    k.node_value = reinterpret_cast<_Float16*>(a->node_value);
    const dim3 grid((k.n + EXPAND_WAVES - 1) / EXPAND_WAVES), block(64 * EXPAND_WAVES);
    if (k.logits_fp32) hipLaunchKernelGGL(expand_kernel<true>, grid, block, 0, (hipStream_t)stream, k);
    else hipLaunchKernelGGL(expand_kernel<false>, grid, block, 0, (hipStream_t)stream, k);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[256];
        snprintf(msg, sizeof(msg), "kernel launch failed: %s", hipGetErrorString(e));
        return fail(BF_ERR_LAUNCH, msg);
    }
    return BF_OK;
}
