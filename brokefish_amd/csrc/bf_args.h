// Shared between the kernel translation units and the host side: layout constants and
// the kernel argument block.  (Design notes follow.)
//
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
//   LayerNorm  per lane half: every 32-wide tile's 16 values form one chain from zero; the tile
//              sums of a quarter of the width are added as a balanced tree (t0 + t1, or
//              (t0 + t1) + (t2 + t3)); the four quarter sums are added in order; then the two halves
//   quantise   s = amax / qmax, q = rint(x / s)  (x / s as a correctly rounded quotient)
//   GEMM       exact int32; descale fl(fl(acc * sa) * sw) + b; several k-chunks are summed
//              in fp64 before the single cast to fp32
//   softmax    exp from bf_exp_neg, p * (1 / l)
// See include/brokefish_hip.h for the blob layouts.

#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "brokefish_hip.h"

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
constexpr int N_SW = 3 * D / 128 + D / 128 + F / 128 + (D / 128) * KCF;   // ffn2: one per (128-row block, k-chunk)
constexpr int LAYER_FLOATS = O_SW + ((N_SW + 3) / 4) * 4;
// a layer's parameters are padded to a whole number of 4 KiB copies (one per workgroup pass)
constexpr int PARAM_BYTES = ((LAYER_FLOATS * 4 + WAVES * FRAG - 1) / (WAVES * FRAG)) * (WAVES * FRAG);
constexpr int PARAM_FLOATS = PARAM_BYTES / 4;
constexpr int LDS_BYTES = RING + 2 * PARAM_BYTES;
constexpr int SW_QKV = 0, SW_OUT = 3 * D / 128, SW_FF1 = SW_OUT + D / 128, SW_FF2 = SW_FF1 + F / 128;
// global side parameters after the layers
constexpr int G_SQ = 0, G_TS = 64 * D, G_CT = G_TS + 12 * D, G_CLOCK = G_CT + 4 * D,
              G_REP = G_CLOCK + 101 * D, G_NFG = G_REP + 3 * D, G_NFB = G_NFG + D,
              GLOBAL_FLOATS = G_NFB + D;

// Layout of the one-position-per-workgroup kernel (bf_board.hip.h), for model width DM: wave w
// owns tiles TW*w .. TW*w+TW-1 of the width.  Per layer a wave streams BPW weight blocks in its
// own consumption order (the feed-forward block in STEPS of 512 hidden channels, of which a wave
// computes four tiles) and reads PW_FLOATS side parameters (part A: attention phase, part B:
// feed-forward phase).  A wave's stream is L * BPW layer blocks, HB head blocks and one block of
// padding (the register prefetch runs one block ahead); see include/brokefish_hip.h.
template <int DM>
struct Layout {
    static constexpr int D = DM, F = 4 * DM, NT = DM / 32, TW = NT / 4, CW = 32 * TW, KC = DM / 256,
                         KCF = F / 256, STEPS = F / 512;
    static constexpr int BPW = 3 * TW * KC + TW * KC + STEPS * (4 * KC + 2 * TW);
    static constexpr int HB = NT / 2;                // head blocks per wave (8 fp32 fragments each)
    static constexpr int SLOTS = DM == 256 ? 3 : 2;  // depth of a wave's private LDS weight ring, in blocks
    static constexpr int A_LN1G = 0, A_LN1B = CW, A_BQ = 2 * CW, A_BK = 3 * CW, A_BV = 4 * CW, A_BOUT = 5 * CW,
                         A_SW = 6 * CW, A_FLOATS = 6 * CW + 16;
    // part B: the first B_LDS_FLOATS are read many times per layer; the tail (first feed-forward
    // bias, 128 * sum(w)) is read once per tile and may be taken from global memory instead of LDS
    static constexpr int B_LN2G = 0, B_LN2B = CW, B_BFF2 = 2 * CW, B_SW = 3 * CW, B_LDS_FLOATS = 3 * CW + 32,
                         B_BFF1 = B_LDS_FLOATS, B_WSUM = B_BFF1 + 128 * STEPS, B_FLOATS = B_WSUM + KCF * CW;
    static constexpr int PW_FLOATS = A_FLOATS + B_FLOATS;
    static constexpr int G_SQ = 0, G_TS = 64 * D, G_CT = G_TS + 12 * D, G_CLOCK = G_CT + 4 * D,
                         G_REP = G_CLOCK + 101 * D, G_NFG = G_REP + 3 * D, G_NFB = G_NFG + D,
                         GLOBAL_FLOATS = G_NFB + D;
};

constexpr int N_PHASES = 12;
// phase slots of the optional cycle profile
enum { PH_EMBED, PH_LN1, PH_QKV, PH_ATTN, PH_OUT, PH_LN2, PH_FF1, PH_FF2, PH_HEADS, PH_STORE, PH_SYNC, PH_TOTAL };

struct KArgs {
    const uint16_t* boards;
    const int16_t* control;
    const uint8_t* rep;
    const uint64_t* mask;
    const uint8_t* active;        // optional [n]: positions with 0 are skipped, their outputs untouched
    const int* leaf_index;        // optional compacted list: slot j of the launch evaluates position leaf_index[j] ...
    const int* leaf_count;        // ... for j < *leaf_count; slots past the count do nothing
    int n;
    const uint8_t* wstream;
    const float* fparams;
    void* policy;
    void* promo;
    float* value;
    int* best;
    int out_fp32, n_layers, l0, l1, n_value;
    int vmode;                    // value head: 0 king row, 1 pooled (mean of the normalised live tokens), 2 prenorm
    float eps;
    float* xpark;                 // workspace: 32 KiB per board slot, residual stream parked during the FFN
    unsigned long long* profile;  // [N_PHASES] cycle sums over waves, profile builds only
    bf_taps taps;
};

// Text returned by bf_last_error() on this thread (set by every translation unit of the library).
void set_error(const char* msg);

// One launcher per separately compiled kernel variant (production, debug taps, phase
// profile); each sets the dynamic-LDS limit once and launches on `stream`.
hipError_t launch_prod(const KArgs& k, int grid, hipStream_t stream);
hipError_t launch_taps(const KArgs& k, int grid, hipStream_t stream);
hipError_t launch_prof(const KArgs& k, int grid, hipStream_t stream);
hipError_t launch_prod_fp8(const KArgs& k, int grid, hipStream_t stream);
hipError_t launch_taps_fp8(const KArgs& k, int grid, hipStream_t stream);
// one position per workgroup (grid = n), for the 256- (int8, e4m3) and the 512-wide network (int8)
hipError_t launch_board256(const KArgs& k, hipStream_t stream);
hipError_t launch_board256_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_board256_fp8(const KArgs& k, hipStream_t stream);
hipError_t launch_board256_fp8_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_board512(const KArgs& k, hipStream_t stream);
hipError_t launch_board512_taps(const KArgs& k, hipStream_t stream);
// the same with two workgroups per compute unit (256-wide network)
hipError_t launch_twin256(const KArgs& k, hipStream_t stream);
hipError_t launch_twin256_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_twin256_fp8(const KArgs& k, hipStream_t stream);
hipError_t launch_twin256_fp8_taps(const KArgs& k, hipStream_t stream);
// one position per workgroup of eight wavefronts (two per quarter of the width), one workgroup
// per compute unit: the lowest latency per position for the 256-wide network (int8, e4m3), and
// the faster form for the 512-wide one (int8)
hipError_t launch_octo256_fp8(const KArgs& k, hipStream_t stream);
hipError_t launch_octo256_fp8_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_octo512(const KArgs& k, hipStream_t stream);
hipError_t launch_octo512_taps(const KArgs& k, hipStream_t stream);
// two positions per workgroup of eight wavefronts (256-wide network): a weight fragment fetched
// once serves both positions
hipError_t launch_duo256(const KArgs& k, hipStream_t stream);
hipError_t launch_duo256_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_duo256_fp8(const KArgs& k, hipStream_t stream);
hipError_t launch_duo256_fp8_taps(const KArgs& k, hipStream_t stream);
// the builds that carry the phase profile
hipError_t launch_twin256_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_octo512_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_duo256_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_board256_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_board512_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_board256_fp8_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_twin256_fp8_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_octo256_fp8_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_duo256_fp8_prof(const KArgs& k, hipStream_t stream);
hipError_t launch_prof_fp8(const KArgs& k, int grid, hipStream_t stream);
// the same kernel with one position per workgroup (the eight-wavefront form for launches that
// cannot fill the GPU): int8, 256-wide network
hipError_t launch_solo256(const KArgs& k, hipStream_t stream);
hipError_t launch_solo256_taps(const KArgs& k, hipStream_t stream);
hipError_t launch_solo256_prof(const KArgs& k, hipStream_t stream);

}  // namespace bf
