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
// lane order is canonical order and an edge's index is a prefix sum over lanes.  Nothing is
// stored per candidate: every pass re-walks the lane's 32 squares from registers, and the
// truncation threshold (the E-th largest log-prior) is found by bisection on the ordered bit
// pattern of the float, so any mask is handled without a candidate buffer.
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

// Three wavefronts per SIMD: left alone the compiler keeps every pass's compares alive side by side
// in 171 registers (two wavefronts per SIMD), and a position's wavefront is a chain of dependent
// steps that only other wavefronts can hide.  168 registers fit without a spill (30 % shorter at
// 65536 positions); at 128 (four wavefronts) 35 registers go to scratch memory, which adds half
// of the kernel's algorithmic bytes again as spill traffic.
__global__ __launch_bounds__(256, 3) void expand_kernel(const KExpand a) {
    const int lane = threadIdx.x & 63;
    int b = blockIdx.x * 4 + (threadIdx.x >> 6);
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

    // this lane's 32 policy logits and its slot's promotion log-probabilities
    float pol[32];
    if (a.logits_fp32) {
        const float* row = (const float*)a.policy + ((size_t)b * 32 + p) * 64 + 32 * half;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const v4f v = *reinterpret_cast<const v4f*>(row + 4 * j);
#pragma unroll
            for (int i = 0; i < 4; i++) pol[4 * j + i] = v[i];
        }
    } else {
        const _Float16* row = (const _Float16*)a.policy + ((size_t)b * 32 + p) * 64 + 32 * half;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const v8h v = *reinterpret_cast<const v8h*>(row + 8 * j);
#pragma unroll
            for (int i = 0; i < 8; i++) pol[8 * j + i] = (float)v[i];
        }
    }
    float lp[4];
    {
        float x[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            x[k] = a.logits_fp32 ? ((const float*)a.promo)[((size_t)b * 32 + p) * 4 + k]
                                 : (float)((const _Float16*)a.promo)[((size_t)b * 32 + p) * 4 + k];
        const float mx = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        const float s = ((__expf(x[0] - mx) + __expf(x[1] - mx)) + __expf(x[2] - mx)) + __expf(x[3] - mx);
        const float ls = __logf(s);
#pragma unroll
        for (int k = 0; k < 4; k++) lp[k] = (x[k] - mx) - ls;
    }
    // visit this lane's candidates in canonical order: f(log-prior, move code)
    auto each = [&](auto&& f) {
#pragma unroll
        for (int i = 0; i < 32; i++) {
            if ((mh >> i) & 1u) {
                const int mv = p * 64 + 32 * half + i;
                if ((pr >> i) & 1u) {
#pragma unroll
                    for (int k = 0; k < 4; k++) f(pol[i] + lp[k], mv | (k << PROMO_SHIFT));
                } else {
                    f(pol[i], mv);
                }
            }
        }
    };

    float mx = -INFINITY;
    each([&](float l, int) { mx = fmaxf(mx, l); });
    mx = wave_max(mx);

    // truncation: T = ordered pattern of the E-th largest log-prior, `need` ties at T survive
    const bool trunc = total > a.E;
    unsigned T = 0;
    int need = 0, tie_before = 0;
    if (trunc) {
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
    float s_all = 0.0f, s_keep = 0.0f;
    each([&](float l, int) {
        const float e = __expf(l - mx);
        s_all += e;
        bool keep = true;
        if (trunc) {
            const unsigned o = ordered(l);
            keep = o > T || (o == T && tie < need);
            tie += o == T;
        }
        if (keep) { kept++; s_keep += e; }
    });
    s_all = wave_sum(s_all);
    s_keep = wave_sum(s_keep);
    int pos = wave_exclusive(kept, lane);
    const int n_edges = __shfl(pos + kept, 63);
    // write the survivors in canonical order
    int16_t* em = a.edge_move + (size_t)b * a.E;
    _Float16* ep = a.edge_prior + (size_t)b * a.E;
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
    hipLaunchKernelGGL(expand_kernel, dim3((k.n + 3) / 4), dim3(256), 0, (hipStream_t)stream, k);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[256];
        snprintf(msg, sizeof(msg), "kernel launch failed: %s", hipGetErrorString(e));
        return fail(BF_ERR_LAUNCH, msg);
    }
    return BF_OK;
}
