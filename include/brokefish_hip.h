/* C-ABI of the MI355X (gfx950) network evaluator: packed board words in, policy /
 * promotion logits and value out, one kernel launch.
 *
 * This is the boundary a host binds in place of the reference's CUDA extension module
 * (reference csrc/encoder.cu:1905-1930 lists the functions that module exports).  Plain
 * pointers and sizes only; every pointer is a DEVICE pointer unless stated otherwise.
 * Nothing here allocates, frees or synchronises: outputs are caller-allocated and the
 * launch is asynchronous on the stream that is passed in.
 *
 * Functions return 0 on success, a negative bf_status on rejected arguments (nothing is
 * launched then) and bf_last_error() describes the most recent failure of the calling
 * thread.
 */
#ifndef BROKEFISH_HIP_H
#define BROKEFISH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum bf_status {
    BF_OK = 0,
    BF_ERR_ARGUMENT = -1,   /* null / misaligned pointer, bad size or mode */
    BF_ERR_UNSUPPORTED = -2, /* network shape this build has no kernel for */
    BF_ERR_LAUNCH = -3,     /* hipLaunchKernel reported an error */
    BF_ERR_DEVICE = -4      /* not a gfx950 device */
};

/* Operand format of the four weight matmuls of every layer.
 *   INT8  exact int32 accumulators; every number of the forward is reproducible bit for bit.
 *   E4M3  OCP e4m3 operands.  Products and sums run on the fp16 matrix instruction, fed with the
 *         operand bytes widened exactly, so a k-tile's accumulator is the exact product to fp32
 *         rounding (the fp8 matrix instructions of gfx950 keep about 16 bits below the largest
 *         addend and are not used). */
enum bf_quant {
    BF_QUANT_INT8 = 0,
    BF_QUANT_E4M3 = 1
};

/* Five kernels compute the same function.
 *   QUAD   four positions per workgroup, one wavefront each, weights shared through LDS
 *          (256-wide network, int8 and e4m3).
 *   BOARD  one position per workgroup, the four wavefronts split the model width; one workgroup
 *          per compute unit: low latency per position (launches that cannot fill the GPU);
 *          both network widths.
 *   TWIN   the BOARD decomposition shaped so that two workgroups share a compute unit (each SIMD
 *          holds two wavefronts that cover each other's waits): the highest throughput
 *          (256-wide network).
 *   OCTO   eight wavefronts per position, one workgroup per compute unit: the lowest latency per
 *          position for the 256-wide network (int8: the DUO kernel with one position per
 *          workgroup; e4m3: the BOARD decomposition with two wavefronts per quarter of the
 *          width), and the faster kernel for the 512-wide one (BOARD decomposition likewise).
 *   DUO    two positions per workgroup of eight wavefronts (the OCTO decomposition, every
 *          wavefront doing its share for both positions), so that a weight fragment fetched from
 *          L2 serves two positions (256-wide network, int8 and e4m3).
 * BOARD, TWIN, OCTO and DUO read the same blobs (board_wstream / board_fparams).  The 256-wide network
 * runs in int8 and e4m3 on all four; the 512-wide network in int8 on OCTO and BOARD.  Kernels that
 * carry a network and a format return bit-identical results for it, so AUTO may pick by batch
 * size: OCTO up to 256 positions, above that DUO (int8) or TWIN (e4m3).  DUO runs in rounds of 512
 * positions; when AUTO has chosen it and the last round would hold at most 256 positions, those
 * are given to the one-position form in a second launch on the same stream (bf_kernel_choice
 * still answers DUO). */
enum bf_kernel {
    BF_KERNEL_AUTO = 0,
    BF_KERNEL_QUAD = 1,
    BF_KERNEL_BOARD = 2,
    BF_KERNEL_TWIN = 3,
    BF_KERNEL_OCTO = 4,
    BF_KERNEL_DUO = 5
};

enum bf_value_mode {
    BF_VALUE_KING = 0,
    BF_VALUE_POOLED = 1,
    BF_VALUE_PRENORM = 2
};

/* Sizes of one 32-token position, fixed by the position format
 * (reference docs/reference/spec.md:94-106). */
#define BF_TOKENS 32
#define BF_POLICY 64
#define BF_PROMO 4

/* Network shape.  Supported: d_model 256, n_heads 8, d_ff 1024 (all kernels, int8 and e4m3)
 * and d_model 512, n_heads 16, d_ff 2048 (BOARD kernel, int8); head width 32, any
 * n_layers >= 1, n_value 1 (tanh scalar) or 3 (loss/draw/win classes). */
typedef struct {
    int32_t d_model, n_layers, n_heads, d_ff, n_value;
    float eps;
} bf_shape;

/* Layout queries for the two parameter blobs of the QUAD kernel (see the layout section at
 * the end of this header).  Return 0 for a shape that kernel does not carry. */
size_t bf_wstream_bytes(const bf_shape* s);   /* int8 weight tiles + fp32 head tiles */
size_t bf_fparams_floats(const bf_shape* s);  /* fp32 / int32 side parameters        */
size_t bf_layer_stride_floats(const bf_shape* s); /* stride of one layer inside fparams */
/* Device scratch the caller lends to a launch of n positions (32 KiB per position, rounded
 * up to a whole workgroup): the kernel parks the fp32 residual stream there while the
 * feed-forward hidden activations occupy the register file.  Contents are meaningless
 * between launches; launches that may overlap need separate workspaces. */
size_t bf_workspace_bytes(const bf_shape* s, int64_t n);
/* The same two blobs in the order of the BOARD and TWIN kernels (the sizes do not depend on
 * the format); 0 for an unsupported shape.  Those kernels need no workspace. */
size_t bf_board_wstream_bytes(const bf_shape* s);
size_t bf_board_fparams_floats(const bf_shape* s);

/* Optional debug outputs ("taps") and teacher forcing.  All pointers may be NULL.
 * B = boards in the call, L = layers run, kc = K / 256.
 * Replaces the reference's debug_stage / forward_stage mechanism
 * (reference brokefish/nn/cuda_impl.py:512-531, csrc/encoder.cu:1575-1598). */
typedef struct {
    const float* x_in;  /* [B,32,d] residual stream to start from instead of the embedding */
    int32_t layer_begin, layer_end; /* run layers [begin, end); 0,0 means all */
    float* embed;       /* [B,32,d]  embedding sum (or x_in echoed)                */
    int8_t* qa_qkv;     /* [B,L,32,d]    operand bytes fed to the QKV matmul       */
    int32_t* acc_qkv;   /* [B,L,kc,32,3d] its int32 accumulators                   */
    int8_t* qa_out;     /* [B,L,32,d]                                              */
    int32_t* acc_out;   /* [B,L,kc,32,d]                                           */
    int8_t* qa_ff1;     /* [B,L,32,d]                                              */
    int32_t* acc_ff1;   /* [B,L,kc,32,d_ff]                                        */
    uint8_t* qa_ff2;    /* [B,L,32,d_ff] unsigned operand bytes of the second FFN matmul */
    int32_t* acc_ff2;   /* [B,L,kc,32,d] accumulators of the unsigned product      */
    float* resid;       /* [B,L,32,d] residual stream after each layer             */
    float* normed;      /* [B,32,d]   after the final LayerNorm                    */
    float* resid_last;  /* [B,32,d]   residual stream after the last layer run: what the
                         * reference's encoder-only call returns
                         * (brokefish/nn/cuda_impl.py:447-463) */
    const int8_t* alive; /* [B,32] non-zero = live token.  Makes the launch encoder-only, as the
                         * reference's encoder_forward (csrc/encoder.cu:1752-1764): x_in and
                         * resid_last are required (they may be the same buffer: in place), the
                         * mask of attention keys comes from here, no board words are read and no
                         * heads run -- boards, control, rep, mask, policy, promo and value of
                         * bf_eval_args are ignored and may be NULL */
} bf_taps;

typedef struct {
    /* inputs (reference csrc/encoder.cu:1770-1790: boards [n,32] int16, control [n]
     * int16, rep [n] uint8, contiguous, on the device) */
    const uint16_t* boards;
    const int16_t* control;
    const uint8_t* rep;
    /* optional legal-move words [n,32], bit s of word p set iff p -> s is legal
     * (reference docs/reference/spec.md:141-143).  NULL = raw logits, as the
     * reference evaluator returns them (docs/reference/spec.md:527-535). */
    const uint64_t* mask;
    int64_t n;
    /* parameters */
    bf_shape shape;
    const uint8_t* wstream;
    const float* fparams;
    /* outputs: policy [n,32,64], promo [n,32,4] in fp16 (out_fp32 = 0, the search
     * contract of reference brokefish/nn/cuda_impl.py:467-472) or fp32; value [n] fp32
     * in [-1,1].  With a mask, illegal policy entries are -inf and best_move [n]
     * (optional) receives slot*64+square of the largest legal logit, lowest index on
     * ties, -1 when no move is legal. */
    void* policy;
    void* promo;
    float* value;
    int32_t* best_move;
    int32_t out_fp32;
    /* operand format of the four weight matmuls: BF_QUANT_INT8 (reference
     * brokefish/nn/quant.py:281-305) or BF_QUANT_E4M3 (quant.py:360-397 with q_max 8,
     * 256-deep k-tiles and 128-row weight blocks, quant.py:82-105).  The parameter blobs
     * must have been packed for the same format. */
    int32_t quant;
    void* workspace;        /* bf_workspace_bytes(shape, n) bytes of device memory (QUAD kernel) */
    size_t workspace_bytes;
    const bf_taps* taps; /* NULL in production */
    /* the weights packed for the BOARD / TWIN kernels (NULL: those kernels are not available
     * to this call); wstream / fparams / workspace may be NULL when QUAD is not to run */
    const uint8_t* board_wstream;
    const float* board_fparams;
    /* optional [n] uint8: positions with 0 are skipped and their outputs left untouched -- the
     * flat leaf staging of the reference's search (brokefish/search/cuda_impl.py:137-145:
     * leaf_board / leaf_control / leaf_rep / leaf_flags) evaluated without compaction and without
     * paying for the leaves that need no evaluation (BOARD / TWIN: the workgroup exits at once;
     * QUAD: the wavefront runs on, storing nothing) */
    const uint8_t* active;
    int32_t kernel;         /* enum bf_kernel; AUTO with the board blobs: OCTO for
                             * n <= bf_board_max_n() and for the 512-wide network, above that
                             * DUO (int8) or TWIN (e4m3); without the board blobs QUAD */
    /* which tokens the value rows read (reference brokefish/nn/model.py:551-617): the king of the
     * side to move (BF_VALUE_KING, the default), the mean of the final-normed live tokens
     * (BF_VALUE_POOLED), or the final norm of the mean of the live tokens' residual stream
     * (BF_VALUE_PRENORM).  The two pooled heads predict in White's frame and the result is negated
     * when Black is to move (control < 0).  BOARD / TWIN / OCTO kernels; QUAD carries the king head. */
    int32_t value_mode;
    /* optional compacted leaf list (see bf_compact_leaves): leaf_index [>= *leaf_count] int32 position
     * numbers and the device-side count.  The launch is sized for n (the size of the flat staging
     * buffers, an upper bound of the count): workgroup j evaluates position leaf_index[j] and
     * workgroups past the count leave at once, so no host round trip is needed to learn how many
     * leaves a simulation step produced.  Inputs are read and outputs written at the position's own
     * row, as with `active` (which must be NULL when a list is given); rows of positions not in the
     * list stay untouched.  Both or neither. */
    const int32_t* leaf_index;
    const int32_t* leaf_count;
} bf_eval_args;

/* Binary interface of this header.  BF_ABI_VERSION is raised whenever a struct or a signature of
 * this header changes; bf_abi_tag() returns (BF_ABI_VERSION << 32) | sizeof(bf_eval_args) as the
 * LIBRARY was compiled.  A binding compiled against this header compares that with its own
 * BF_ABI_TAG before its first call and refuses a library it was not built for (a shorter
 * bf_eval_args would make the library read pointers from beyond the caller's struct).  No
 * counterpart in the reference, whose module and kernels are one compilation. */
#define BF_ABI_VERSION 6
#define BF_ABI_TAG (((uint64_t)BF_ABI_VERSION << 32) | (uint64_t)sizeof(bf_eval_args))
uint64_t bf_abi_tag(void);

/* Largest n for which AUTO prefers OCTO over DUO / TWIN on the 256-wide network. */
int64_t bf_board_max_n(void);
/* The kernel AUTO would run for these arguments (enum bf_kernel), or a negative bf_status. */
int bf_kernel_choice(const bf_eval_args* args);

/* The evaluator.  Replaces model_forward of the reference extension
 * (reference csrc/encoder.cu:1770-1876, bound at :1918-1925; called from
 * brokefish/nn/cuda_impl.py:497-503).  `stream` is a hipStream_t (NULL = default). */
int bf_model_forward(const bf_eval_args* args, void* stream);

/* The evaluator for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as bf_model_forward on the QUAD kernel (args->kernel must be
 * BF_KERNEL_QUAD or BF_KERNEL_AUTO; wstream / fparams required), except that args->workspace and
 * args->workspace_bytes are ignored: the kernel's workspace is a static device array of
 * BF_STATIC_MAX_N * 32 KiB inside the library, which every GPU the library runs on holds until
 * the process ends.  n above BF_STATIC_MAX_N is rejected with BF_ERR_ARGUMENT.  The call makes
 * no hipMalloc / hipFree; its first call on a device looks the array's address up (so make one
 * call per device before capturing).  All calls on one GPU share that GPU's array: calls that
 * may overlap on one GPU (two streams, two threads) race -- serialise them or use
 * bf_model_forward with separate workspaces.  Nothing in the array has to start at zero. */
#define BF_STATIC_MAX_N 1024
int bf_model_forward_static(const bf_eval_args* args, void* stream);

/* Quantisation maxima of the signed / unsigned activation formats, for the host to pin
 * against its own constants.  Replaces int8_q_max (reference csrc/encoder.cu:1926-1929). */
void bf_int8_q_max(double* s8, double* u8);

/* The value a row's (and a weight block's) largest magnitude is mapped to in the e4m3
 * format.  Replaces fp8_q_max (reference csrc/encoder.cu:1905-1930; pinned against
 * brokefish/nn/quant.py:105). */
double bf_fp8_q_max(void);

/* Message for the last non-zero status returned to this thread. */
const char* bf_last_error(void);

/* Average device time of the evaluator kernel, measured with HIP events recorded on
 * `stream` around `iters` back-to-back launches (after `warmup` launches).  Returns
 * milliseconds per launch, or a negative bf_status.  Synchronises the stream.
 * Stands in for the reference's in-kernel phase profile hooks
 * (reference csrc/encoder.cu:1886-1903) at whole-kernel granularity. */
double bf_time_kernel_ms(const bf_eval_args* args, void* stream, int warmup, int iters);

/* Measured rate of the matrix pipe, in TOP/s: a register-resident loop of independent
 * 32x32 MFMA chains (v_mfma_i32_32x32x32_i8 for BF_QUANT_INT8; v_mfma_f32_32x32x16_f16 for
 * BF_QUANT_E4M3, whose operands the kernels widen exactly to fp16), two wavefronts per SIMD on every compute unit, no memory traffic inside the
 * loop; `iters` chain steps per wavefront, `reps` timed launches after one warm-up launch.
 * `scratch` is a 16-byte aligned DEVICE buffer of 4096 zero bytes.  Returns a negative
 * bf_status on error.  Synchronises the stream.  The evaluator's roofline is quoted against
 * the datasheet peak; this number says how much of that peak the instruction the kernels use
 * reaches on the installed part.  Follows the reference's own ceiling measurement (reference
 * docs/ledger/perf.md:616-642). */
double bf_mfma_rate(int quant, int* scratch, int iters, int reps, void* stream);

/* Measured rate, in TB/s, at which the compute units can stream one buffer out of the cache
 * hierarchy when every workgroup reads all of it -- the access pattern of the evaluator's weights
 * (each position's workgroup reads the whole network; the kernels' weight traffic is priced
 * against this number).  `workgroups` workgroups of four wavefronts each read `bytes` (a multiple
 * of 32768) from the DEVICE buffer `buf`, wavefront w its quarter, 16 bytes per lane and load,
 * eight loads in flight, from staggered starting offsets; `reps` timed launches after one
 * warm-up launch; `sink` is a DEVICE buffer of 256 bytes that is never written for a buffer of
 * equal 32-bit words.  Returns a negative bf_status on error.  Synchronises the stream.
 * No counterpart in the reference. */
double bf_stream_rate(const void* buf, size_t bytes, int workgroups, int reps, int* sink, void* stream);

/* The kernels' row quantisers on their own, for tests: out[i] = the byte the evaluator would write
 * for x[i] under the activation scale `scale` (n a multiple of 4, x 16-byte aligned DEVICE memory).
 *   BF_PROBE_S8       signed int8: rint(x / scale) as a correctly rounded quotient, low byte kept
 *                     (the row scale keeps |x / scale| <= 127; nothing clamps here)
 *   BF_PROBE_U8_RELU  the unsigned quantiser of the feed-forward hidden row with the ReLU folded
 *                     in: rint(max(x, 0) / scale) saturated to [0, 255]
 *   BF_PROBE_E4M3     OCP e4m3 code of x / scale clamped to +-448
 * The device twin of the reference's quantiser unit tests (reference csrc/tests/tint8.cu:39-61,
 * :190-227).  Asynchronous on `stream`. */
enum bf_probe_mode { BF_PROBE_S8 = 0, BF_PROBE_U8_RELU = 1, BF_PROBE_E4M3 = 2 };
int bf_quant_probe(int mode, const float* x, float scale, int64_t n, uint8_t* out, void* stream);

/* In-kernel phase accounting, the counterpart of the reference's profile hooks
 * (reference csrc/encoder.cu:1083-1177 and :1886-1903: set_profile / read_profile /
 * profile_phases).  bf_profile_phases runs a separately compiled build of the kernel the
 * arguments select (every kernel, both formats, both widths) that reads the shader clock at
 * phase boundaries and ADDS, per wavefront, the cycles of each phase into
 * cycles[bf_profile_phase_count()] (DEVICE memory, zeroed by the caller before the first launch
 * it wants counted: several launches accumulate, as the reference's set_profile / read_profile
 * pair does): divide by the wavefronts of the launches (BOARD and TWIN 4 n, OCTO 8 n, DUO
 * 8 ceil(n / 2), QUAD 4 ceil(n / 4)).  Slot "sync_wait" is the time spent waiting at workgroup barriers (QUAD:
 * at the synchronisations of the LDS weight ring) and is also contained in the enclosing phases;
 * slot "total" is the wavefront lifetime.  In the one-position-per-workgroup kernels the matrix
 * products of a head are issued inside "qkv_gemm_epilogue" and those of the out-projection and
 * feed-forward tiles inside their phases; "store" is the policy / promotion / value output.
 * The production kernels carry none of this code. */
int bf_profile_phases(const bf_eval_args* args, void* stream, uint64_t* cycles);
int bf_profile_phase_count(void);
const char* bf_profile_phase_name(int i);

/* Edge expansion behind the evaluator: turns the logits of n positions and their legal-move
 * words into the edges of search nodes, on the device, with no host round trip.  Replaces the
 * expand step of the reference's search (reference docs/reference/search.md:616-636;
 * brokefish/search/torch_impl.py:962-1033; device twin csrc/search.cuh:540-798).
 *
 * Per position: the set bits of the 32 mask words are enumerated in canonical order (ascending
 * slot, then square; a move of a live pawn onto the last rank of the side to move -- rank 8 when
 * control > 0, rank 1 when control < 0 -- gives four edges in the order N B R Q).  An edge's
 * log-prior is policy[slot][square], plus log_softmax(promo[slot])[type] for a promotion edge.
 * If there are more than max_edges candidates the max_edges largest are kept (ties by canonical
 * order; the survivors stay in canonical order).  edge_prior is the softmax over the survivors.
 *   edge_move  [n, max_edges] int16   slot*64+square | type << 11; 0 beyond n_edges
 *   edge_prior [n, max_edges] fp16    0 beyond n_edges
 *   n_edges    [n] int32; count [n] int32 (candidates before truncation, optional);
 *   dropped    [n] fp32 (prior mass removed by the truncation, optional);
 *   node_value [n] fp16 = (value + 1) / 2 (optional; needs value).
 * active (optional, [n] uint8): positions with 0 are left untouched.  policy / promo are the
 * evaluator's outputs: fp16, or fp32 when logits_fp32 is set; policy may be raw or already
 * masked (only legal entries are read).  A position with no legal move gets n_edges = 0. */
typedef struct {
    const void* policy;
    const void* promo;
    const float* value;
    const uint64_t* mask;
    const uint16_t* boards;
    const int16_t* control;
    const uint8_t* active;
    int64_t n;
    int32_t max_edges;      /* 1 .. 255 (the reference's E, 96 by default) */
    int32_t logits_fp32;
    int16_t* edge_move;
    void* edge_prior;
    int32_t* n_edges;
    int32_t* count;
    float* dropped;
    void* node_value;
    /* optional compacted leaf list, as in bf_eval_args (then `active` must be NULL) */
    const int32_t* leaf_index;
    const int32_t* leaf_count;
} bf_expand_args;

int bf_expand(const bf_expand_args* args, void* stream);

/* Compaction of the search's leaf flags into the list the evaluator and the expansion take: writes
 * the numbers of the positions whose flag is non-zero, in ascending order, to leaf_index[0 .. count)
 * and the count to leaf_count[0] (both DEVICE memory; leaf_index holds n entries, entries past the
 * count are left as they were).  The "compacted list plus a count" of the reference's design
 * retrospective (reference docs/journal/2026-08-09-kernel-design-retrospective.md:140-154) over its
 * flat staging (brokefish/search/cuda_impl.py:137-145: leaf_flags).  One workgroup; asynchronous. */
int bf_compact_leaves(const uint8_t* flags, int64_t n, int32_t* leaf_index, int32_t* leaf_count, void* stream);

/* Legal-move words on the device.  Replaces env.movegen of the reference (reference
 * docs/reference/spec.md:152-172; brokefish/env/torch_impl.py:251-289): for each of n positions
 * (boards [n,32] uint16, control [n] int16) writes mask [n,32] uint64 -- bit s of word p set iff
 * slot p may legally move to square s (spec.md:141-143) -- and, if in_check is not NULL, whether
 * the side to move is in check.  Positions are assumed well formed (spec.md:108-116: both kings
 * alive in slots 15 and 31).  Asynchronous on `stream`. */
int bf_movegen(const uint16_t* boards, const int16_t* control, int64_t n, uint64_t* mask,
               uint8_t* in_check, void* stream);

/* -------------------------------------------------------------------------------------
 * Blob layouts (what the host packer writes; brokefish_amd/hip_impl.py is the packer).
 *
 * Lane order: within a 32-wide tile, lane half g (0/1) and index r (0..15) address
 *     ch(r, g) = 8 * (r / 4) + 4 * g + (r % 4).
 *
 * wstream: a sequence of 1 KiB fragments; a fragment holds 64 lanes x 16 bytes.  For an
 * int8 fragment of output tile n and k-step s of matrix W [N, K] (rows = output
 * channels), lane = 32 * g + o holds W[32 n + o][k0 + 32 s + ch(r, g)] at byte r.
 * 8 fragments (s = 0..7, one 256-wide k-chunk) make a block; per layer the blocks are
 *     for head h:  Q tile h, K tile h, V tile h        (rows h*32, d + h*32, 2d + h*32)
 *     out-proj tiles 0..7
 *     ffn1 tiles 0..31
 *     for ffn2 output tile n: for k-chunk c = 0..3: block (n, c)
 * In the e4m3 format the bytes are OCP e4m3 codes instead of int8 values, in the same
 * order; each weight scale then covers a 128-row x 256-deep block, wsum is all zero.
 * After the last layer three 32 KiB fp32 head tiles: head tile m (rows 32m..32m+31
 * of [policy(64); promo(4); value(n_value); zeros]), fragment (n, q), lane 32g + o holds
 * the four floats W[32 m + o][32 n + 8 q + 4 g + 0..3].
 *
 * BOARD / TWIN kernel blobs.  Wave w of a workgroup owns tiles TW*w .. TW*w+TW-1 of the model
 * width (TW = d/128), kc = d/256, steps = d_ff/512.  board_wstream is, for each wave w, its own
 * stream: per layer the 8 KiB blocks (same fragment format as above)
 *     for own head i: Q tile chunks 0..kc-1, K tile chunks, V tile chunks
 *     out-proj: for own tile i: chunks 0..kc-1
 *     for step s: ffn1: for i = 0..3: hidden tile 16 s + 4 w + i, chunks 0..kc-1;
 *                 ffn2: for chunk c = 2 s, 2 s + 1: for own tile i: block (tile, c)
 * then d/64 blocks holding head tile w (the fp32 fragments (n, q) in order; zeros for w = 3)
 * and one block of zeros (the weight prefetch reads one block past a wave's last).
 * board_fparams is, for each wave w, per layer: part A  ln1_gamma ln1_beta b_q b_k b_v b_out
 * (own channels, d/4 each) sw_q[TW] sw_k[TW] sw_v[TW] sw_out[TW] (per own tile, padded to 16);
 * part B  ln2_gamma ln2_beta b_ffn2 (own channels) sw_ffn1[4 per step, padded to 16] sw_ffn2[TW]
 * (padded to 16; in the e4m3 format sw_ffn2[TW][d_ff/256], one per own tile and k-chunk)
 * b_ffn1 (own hidden channels: 128 per step) wsum[d_ff/256][d/4] (int32, own channels; all zero
 * in the e4m3 format); after the four waves the embedding tables and norm_f as below.
 *
 * fparams (fp32 unless noted), per layer at stride bf_layer_stride_floats() (the layer's
 * parameters zero-padded to a multiple of 4 KiB, because a workgroup copies them to LDS
 * in 4 KiB passes):
 *     ln1_gamma[d] ln1_beta[d] b_qkv[3d] b_out[d] ln2_gamma[d] ln2_beta[d] b_ffn1[f]
 *     b_ffn2[d] wsum[kc_f][d] (int32: 128 * sum of the int8 weights of ffn2 row over
 *     k-chunk c) sw_qkv[3d/128] sw_out[d/128] sw_ffn1[f/128] sw_ffn2[d/128][kc_f]
 *     (weight scales per 128 output rows; ffn2 carries one per k-chunk, which the int8
 *     format fills with the same value four times)
 * then the five embedding tables (square 64, type_special 12, color_turn 4, clock 101,
 * rep 3 rows of d) and norm_f gamma[d], beta[d].
 * ----------------------------------------------------------------------------------- */

#ifdef __cplusplus
}
#endif
#endif
