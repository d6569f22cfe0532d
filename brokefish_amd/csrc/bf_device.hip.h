// Device helpers shared by the evaluator kernels: vector types, lane exchange, exp / tanh,
// program-order anchors, the MFMA block product and the quantisers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <type_traits>

#include "bf_args.h"

typedef long v2l __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

namespace bf {


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

// Program-order anchors: an empty volatile asm that reads and writes a register forces the
// value to exist at this point, so the compiler cannot postpone a tile's epilogue past the
// following tiles (which would keep every accumulator alive and spill it).
__device__ __forceinline__ void pin(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(double& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(int& v) { asm volatile("" : "+v"(v)); }

__device__ __forceinline__ void pin16(float (&v)[16]) {
#pragma unroll
    for (int i = 0; i < 16; i++) pin(v[i]);
}

__device__ __forceinline__ v4f ldg4(const float* p) { return *reinterpret_cast<const v4f*>(p); }
__device__ __forceinline__ v4i ldg4i(const float* p) { return *reinterpret_cast<const v4i*>(p); }
// the 16 per-channel parameters a lane needs for one 32-wide tile starting at p
__device__ __forceinline__ void load_tile16(const float* p, int g, v4f (&b)[4]) {
#pragma unroll
    for (int j = 0; j < 4; j++) b[j] = ldg4(p + 8 * j + 4 * g);
}
__device__ __forceinline__ void load_tile16i(const float* p, int g, v4i (&b)[4]) {
#pragma unroll
    for (int j = 0; j < 4; j++) b[j] = ldg4i(p + 8 * j + 4 * g);
}

// Eight e4m3 bytes (byte j of `bytes` = this lane's k index j) as eight fp16 values.  Exact:
// every e4m3 value, subnormals included, is an fp16 value.
__device__ __forceinline__ v8h e4m3x8_as_f16(long bytes) {
    const unsigned lo = (unsigned)bytes, hi = (unsigned)((unsigned long)bytes >> 32);
    const v2h a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
    const v2h b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
    const v2h c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
    const v2h d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
    return v8h{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// One 16-deep step of an e4m3 block product.  The operands go through the fp16 matrix
// instruction: its products are exact (two 4-bit significands) and its adder carries fp32
// precision, where v_mfma_f32_32x32x16_fp8_fp8 aligns the 16 products to the largest and keeps
// only about 16 bits below it.  Lane / k pairing is the same for both instructions (lane (i, g)
// holds k = 8g .. 8g+7), so the byte packing does not change.
template <bool SWAP>
__device__ __forceinline__ v16f e4m3_step(long w, long act, v16f acc) {
    const v8h wh = e4m3x8_as_f16(w), ah = e4m3x8_as_f16(act);
    return SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, wh, acc, 0, 0, 0)
                : __builtin_amdgcn_mfma_f32_32x32x16_f16(wh, ah, acc, 0, 0, 0);
}

// acc[out_channel r][token] (weights as A) or acc[token r][out_channel] (SWAP, weights as B).
// int8: eight v_mfma_i32_32x32x32_i8; e4m3: each 16-byte fragment is two 16-deep steps.
template <bool FP8> struct Acc { typedef v16i type; };
template <> struct Acc<true> { typedef v16f type; };

template <bool SWAP, bool FP8>
__device__ __forceinline__ typename Acc<FP8>::type mfma8(const v4i (&w)[8], const v4i (&act)[8]) {
    if constexpr (FP8) {
        v16f acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const v2l wl = __builtin_bit_cast(v2l, w[s]);
            const v2l al = __builtin_bit_cast(v2l, act[s]);
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) acc = e4m3_step<SWAP>(wl[hlf], al[hlf], acc);
        }
        return acc;
    } else {
        v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 8; s++)
            acc = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(act[s], w[s], acc, 0, 0, 0)
                       : __builtin_amdgcn_mfma_i32_32x32x32_i8(w[s], act[s], acc, 0, 0, 0);
        return acc;
    }
}

// accumulator element as fp32 (exact for the int32 accumulators: they stay below 2^24)
__device__ __forceinline__ float accf(const v16i& a, int i) { return (float)a[i]; }
__device__ __forceinline__ float accf(const v16f& a, int i) { return a[i]; }
__device__ __forceinline__ int accbits(const v16i& a, int i) { return a[i]; }
__device__ __forceinline__ int accbits(const v16f& a, int i) { return __float_as_int(a[i]); }

// m / 127 and m / 255 (the activation scales), correctly rounded for every finite m: the
// reciprocal constant and two fused corrections.  Equal to IEEE division on all 2^31 positive
// floats, subnormals included (checked exhaustively on the CPU), and a third of its instructions.
__device__ __forceinline__ float div127(float m) {
    const float c = 1.0f / 127.0f;
    const float q = m * c;
    return __builtin_fmaf(__builtin_fmaf(-q, 127.0f, m), c, q);
}
__device__ __forceinline__ float div255(float m) {
    const float c = 1.0f / 255.0f;
    const float q = m * c;
    return __builtin_fmaf(__builtin_fmaf(-q, 255.0f, m), c, q);
}

// ---- row operations -------------------------------------------------------------------

// four quotients v / sa (correctly rounded) -> one packed dword.
// int8: round to nearest even, low bytes gathered.  e4m3: clamp to the format's range and
// convert with the hardware's round-to-nearest-even OCP e4m3 conversion.
template <bool FP8>
__device__ __forceinline__ unsigned quant4(float v0, float v1, float v2, float v3, float sa, float inv) {
    float qf[4];
    const float v[4] = {v0, v1, v2, v3};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // correctly rounded v / sa from the reciprocal and two fused corrections
        const float q0 = v[i] * inv;
        const float rem = __builtin_fmaf(-q0, sa, v[i]);
        qf[i] = __builtin_fmaf(rem, inv, q0);
    }
    if constexpr (FP8) {
#pragma unroll
        for (int i = 0; i < 4; i++) qf[i] = __builtin_fminf(__builtin_fmaxf(qf[i], -448.0f), 448.0f);
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(qf[0], qf[1], 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(qf[2], qf[3], w, true);
        return (unsigned)w;
    } else {
        // Adding 1.5 * 2^23 rounds to nearest even and leaves the integer in the low bits of the sum;
        // the sub-dword form of the add writes that low byte straight into its place in the packed
        // dword (held against rint on the host, ties included, by tests/test_quantiser_gpu.py).
        const float magic = 12582912.0f;
        unsigned w;
        asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD" : "=v"(w) : "v"(qf[0]), "v"(magic));
        asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(qf[1]), "v"(magic));
        asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(qf[2]), "v"(magic));
        asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(qf[3]), "v"(magic));
        return w;
    }
}

// The unsigned int8 quantiser of the feed-forward hidden row with the ReLU folded in: four
// correctly rounded quotients v / sa, converted with v_cvt_pk_u8_f32 -- round to nearest even,
// saturating to [0, 255], so a negative input gives 0 exactly as max(v, 0) would (held against
// rint + clamp on the host, every tie k + 0.5 included, by tests/test_quantiser_gpu.py) -- each
// conversion writing its own byte of the dword.
__device__ __forceinline__ unsigned quant4_relu_u8(float v0, float v1, float v2, float v3, float sa, float inv) {
    const float v[4] = {v0, v1, v2, v3};
    unsigned w = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float q0 = v[i] * inv;
        const float rem = __builtin_fmaf(-q0, sa, v[i]);
        w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(rem, inv, q0), i, w);
    }
    return w;
}

// signed quantiser (int8: amax -> 127, e4m3: amax -> 8) of one token row spread over two
// lanes; y is [tiles][16]
template <int NTILES, bool FP8>
__device__ __forceinline__ void quant_s8(const float (&y)[NTILES][16], int g, v4i (&q)[NTILES], float& sa) {
    float am = 0.0f;
#pragma unroll
    for (int n = 0; n < NTILES; n++)
#pragma unroll
        for (int r = 0; r < 16; r++) am = __builtin_fmaxf(am, __builtin_fabsf(y[n][r]));
    am = __builtin_fmaxf(am, partner(am, g));
    sa = am > 0.0f ? (FP8 ? am * 0.125f : div127(am)) : 1.0f;
    const float inv = 1.0f / sa;
#pragma unroll
    for (int n = 0; n < NTILES; n++)
#pragma unroll
        for (int j = 0; j < 4; j++)
            q[n][j] = (int)quant4<FP8>(y[n][4 * j], y[n][4 * j + 1], y[n][4 * j + 2], y[n][4 * j + 3], sa, inv);
}

}  // namespace bf
