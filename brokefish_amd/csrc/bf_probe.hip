// Matrix-pipe rate probe: a register-resident loop of independent MFMA chains with no memory
// traffic inside the loop, so a measured ceiling stands next to the datasheet peak the
// evaluator's roofline is quoted against.  Same method as the reference's own ceiling
// measurement (reference docs/ledger/perf.md:616-642: raw mma in a register-resident loop with
// eight independent accumulators).
//
// Every wavefront keeps four independent 32x32 accumulators and issues them round-robin; two
// wavefronts per SIMD give eight chains in flight per matrix pipe.  Operands are read once from
// `scratch` (so nothing folds to a constant) and the accumulators are stored back only under a
// condition the data never meets, which keeps the loop alive without a store in it.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "bf_args.h"

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int CHAINS = 4;
constexpr int PROBE_THREADS = 256;

template <bool FP8>
__global__ __launch_bounds__(PROBE_THREADS) void mfma_loop(int* scratch, int iters) {
    const int lane = threadIdx.x & 63;
    const v4i a = *reinterpret_cast<const v4i*>(scratch + 4 * lane);
    const v4i b = *reinterpret_cast<const v4i*>(scratch + 256 + 4 * lane);
    int fold = 0;
    if constexpr (FP8) {
        // the e4m3 kernels feed their operands, widened exactly, to the fp16 instruction
        const v8h ah = __builtin_bit_cast(v8h, a), bh = __builtin_bit_cast(v8h, b);
        v16f acc[CHAINS];
#pragma unroll
        for (int c = 0; c < CHAINS; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[c][i] = 0.0f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int c = 0; c < CHAINS; c++) {
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, acc[c], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bh, ah, acc[c], 0, 0, 0);
            }
        }
#pragma unroll
        for (int c = 0; c < CHAINS; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) fold ^= __float_as_int(acc[c][i]);
    } else {
        v16i acc[CHAINS];
#pragma unroll
        for (int c = 0; c < CHAINS; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[c][i] = 0;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int c = 0; c < CHAINS; c++)
                acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < CHAINS; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) fold ^= acc[c][i];
    }
    // zero operands give zero accumulators: this store never happens on the probe's own input
    if (fold == 0x5bd1e995) scratch[512 + lane] = fold;
}

// Weight-stream probe: every workgroup reads the whole buffer once, as a position's workgroup
// reads the whole network -- wavefront w its quarter, 16 bytes per lane and load, eight loads in
// flight, nothing else in the loop.  Workgroups start at different offsets of their quarters
// (they are at different layers in the evaluator too) and wrap around.
constexpr int STREAM_AHEAD = 8;
__global__ __launch_bounds__(PROBE_THREADS) void stream_loop(const uint8_t* buf, size_t chunks_per_quarter, int* sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t* base = buf + (size_t)wave * chunks_per_quarter * 1024 + lane * 16;
    const size_t start = ((size_t)blockIdx.x * 2654435761u) % chunks_per_quarter;
    v4i acc = {0, 0, 0, 0};
    for (size_t c = 0; c < chunks_per_quarter; c += STREAM_AHEAD) {
        v4i v[STREAM_AHEAD];
#pragma unroll
        for (int u = 0; u < STREAM_AHEAD; u++) {
            size_t idx = start + c + u;
            if (idx >= chunks_per_quarter) idx -= chunks_per_quarter;
            v[u] = *reinterpret_cast<const v4i*>(base + idx * 1024);
        }
#pragma unroll
        for (int u = 0; u < STREAM_AHEAD; u++) acc ^= v[u];
    }
    // keeps the loads alive; never true for a buffer of equal 32-bit words (the xor of an even count is 0)
    if ((acc[0] ^ acc[1]) == 0x5bd1e995 && (acc[2] ^ acc[3]) == 0x1b873593) sink[lane] = acc[0];
}

}  // namespace

extern "C" double bf_mfma_rate(int quant, int* scratch, int iters, int reps, void* stream) {
    auto fail = [](int code, const char* msg) {
        bf::set_error(msg);
        return (double)code;
    };
    if (quant != BF_QUANT_INT8 && quant != BF_QUANT_E4M3) return fail(BF_ERR_ARGUMENT, "quant must be BF_QUANT_INT8 or BF_QUANT_E4M3");
    if (!scratch || ((uintptr_t)scratch & 15)) return fail(BF_ERR_ARGUMENT, "scratch must be a 16-byte aligned device buffer of 4096 zero bytes");
    if (iters < 1 || iters > (1 << 24) || reps < 1 || reps > 1000) return fail(BF_ERR_ARGUMENT, "iters must be in [1, 2^24] and reps in [1, 1000]");
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
        return fail(BF_ERR_LAUNCH, "cannot read the compute-unit count");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(2 * cus), block(PROBE_THREADS);     // two wavefronts per SIMD
    auto go = [&]() {
        if (quant == BF_QUANT_E4M3) hipLaunchKernelGGL(mfma_loop<true>, grid, block, 0, s, scratch, iters);
        else hipLaunchKernelGGL(mfma_loop<false>, grid, block, 0, s, scratch, iters);
    };
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    }
    go();                                               // warm-up: code load and clock ramp
    (void)hipEventRecord(e0, s);
    for (int r = 0; r < reps; r++) go();
    (void)hipEventRecord(e1, s);
    const hipError_t e = hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    const hipError_t le = hipGetLastError();
    if (e != hipSuccess || le != hipSuccess) return fail(BF_ERR_LAUNCH, hipGetErrorString(e != hipSuccess ? e : le));
    // 2*32*32*32 operations per int8 instruction; the e4m3 chain step is two 32x32x16 fp16 instructions
    const double ops = 65536.0 * CHAINS * (double)iters * (PROBE_THREADS / 64) * grid.x * reps;
    return ops / ((double)ms * 1e-3) / 1e12;
}

extern "C" double bf_stream_rate(const void* buf, size_t bytes, int workgroups, int reps, int* sink, void* stream) {
    auto fail = [](int code, const char* msg) {
        bf::set_error(msg);
        return (double)code;
    };
    constexpr size_t UNIT = (size_t)4 * STREAM_AHEAD * 1024;   // four quarters of whole groups of loads
    if (!buf || ((uintptr_t)buf & 15) || !sink) return fail(BF_ERR_ARGUMENT, "buf must be a 16-byte aligned device buffer and sink 256 device bytes");
    if (bytes < UNIT || bytes % UNIT) return fail(BF_ERR_ARGUMENT, "bytes must be a positive multiple of 32768");
    if (workgroups < 1 || workgroups > (1 << 20) || reps < 1 || reps > 1000) return fail(BF_ERR_ARGUMENT, "workgroups must be in [1, 2^20] and reps in [1, 1000]");
    hipStream_t s = (hipStream_t)stream;
    auto go = [&]() { hipLaunchKernelGGL(stream_loop, dim3(workgroups), dim3(PROBE_THREADS), 0, s, (const uint8_t*)buf, bytes / 4096, sink); };
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    }
    go();                                               // warm-up: the buffer into the caches
    (void)hipEventRecord(e0, s);
    for (int r = 0; r < reps; r++) go();
    (void)hipEventRecord(e1, s);
    const hipError_t e = hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    const hipError_t le = hipGetLastError();
    if (e != hipSuccess || le != hipSuccess) return fail(BF_ERR_LAUNCH, hipGetErrorString(e != hipSuccess ? e : le));
    return (double)bytes * workgroups * reps / ((double)ms * 1e-3) / 1e12;
}

// ---- quantiser probe ---------------------------------------------------------------------------
// The kernels' row quantisers applied to a caller's values with a caller's scale, so that the
// instruction sequences they are built from (the corrected-reciprocal quotient, the byte-select
// add, v_cvt_pk_u8_f32, the e4m3 conversion) can be held against rint / clamp on the host.
#include "bf_device.hip.h"

namespace {

template <int MODE>
__global__ void quant_probe(const float* x, float scale, long n4, unsigned* out) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const float4 v = reinterpret_cast<const float4*>(x)[i];
    const float inv = 1.0f / scale;
    unsigned w;
    if constexpr (MODE == BF_PROBE_S8) w = bf::quant4<false>(v.x, v.y, v.z, v.w, scale, inv);
    else if constexpr (MODE == BF_PROBE_U8_RELU) w = bf::quant4_relu_u8(v.x, v.y, v.z, v.w, scale, inv);
    else w = bf::quant4<true>(v.x, v.y, v.z, v.w, scale, inv);
    out[i] = w;
}

}  // namespace

extern "C" int bf_quant_probe(int mode, const float* x, float scale, int64_t n, uint8_t* out, void* stream) {
    if (!x || !out || n < 4 || (n & 3) || ((uintptr_t)x & 15) || ((uintptr_t)out & 3) || !(scale > 0.0f)) {
        bf::set_error("bf_quant_probe: x (16-byte aligned) and out (4-byte aligned) must not be NULL, n a positive multiple of 4, scale > 0");
        return BF_ERR_ARGUMENT;
    }
    const long n4 = n / 4;
    const dim3 grid((unsigned)((n4 + 255) / 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    unsigned* o = reinterpret_cast<unsigned*>(out);
    if (mode == BF_PROBE_S8) hipLaunchKernelGGL(quant_probe<BF_PROBE_S8>, grid, block, 0, s, x, scale, n4, o);
    else if (mode == BF_PROBE_U8_RELU) hipLaunchKernelGGL(quant_probe<BF_PROBE_U8_RELU>, grid, block, 0, s, x, scale, n4, o);
    else if (mode == BF_PROBE_E4M3) hipLaunchKernelGGL(quant_probe<BF_PROBE_E4M3>, grid, block, 0, s, x, scale, n4, o);
    else {
        bf::set_error("bf_quant_probe: mode must be BF_PROBE_S8, BF_PROBE_U8_RELU or BF_PROBE_E4M3");
        return BF_ERR_ARGUMENT;
    }
    if (hipGetLastError() != hipSuccess) {
        bf::set_error("bf_quant_probe: launch failed");
        return BF_ERR_LAUNCH;
    }
    return BF_OK;
}
