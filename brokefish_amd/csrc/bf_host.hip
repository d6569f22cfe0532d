// Host side of the evaluator library: the C-ABI of include/brokefish_hip.h.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <atomic>
#include <cstring>
#include <mutex>

#include "bf_args.h"



static thread_local char g_err[512] = "";

static int fail(int code, const char* msg) {
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return code;
}

void bf::set_error(const char* msg) { snprintf(g_err, sizeof(g_err), "%s", msg); }

static bool shape_ok(const bf_shape* s) {   // the four-positions-per-workgroup kernel
    return s && s->d_model == bf::D && s->d_ff == bf::F && s->n_heads == bf::NH && s->n_layers >= 1 &&
           (s->n_value == 1 || s->n_value == 3);
}

static bool shape512(const bf_shape* s) {
    return s && s->d_model == 512 && s->d_ff == 2048 && s->n_heads == 16 && s->n_layers >= 1 &&
           (s->n_value == 1 || s->n_value == 3);
}

static bool board_shape_ok(const bf_shape* s) { return shape_ok(s) || shape512(s); }

// AUTO runs one workgroup of eight wavefronts per compute unit (lowest latency per position) up
// to this many positions, which is one per compute unit of an MI355X; above it, the forms built
// for throughput (256-wide network): two positions per workgroup (int8) or two workgroups of
// four wavefronts per compute unit (e4m3).
static const int64_t kBoardMaxN = 256;

template <int DM>
static size_t board_wstream_bytes(int n_layers) {
    typedef bf::Layout<DM> L;
    return (size_t)4 * ((size_t)n_layers * L::BPW + L::HB + 1) * bf::BLOCK;
}
template <int DM>
static size_t board_fparams_floats(int n_layers) {
    typedef bf::Layout<DM> L;
    return (size_t)4 * n_layers * L::PW_FLOATS + L::GLOBAL_FLOATS;
}

extern "C" size_t bf_board_wstream_bytes(const bf_shape* s) {
    if (shape_ok(s)) return board_wstream_bytes<256>(s->n_layers);
    if (shape512(s)) return board_wstream_bytes<512>(s->n_layers);
    return 0;
}

extern "C" size_t bf_board_fparams_floats(const bf_shape* s) {
    if (shape_ok(s)) return board_fparams_floats<256>(s->n_layers);
    if (shape512(s)) return board_fparams_floats<512>(s->n_layers);
    return 0;
}

extern "C" int64_t bf_board_max_n(void) { return kBoardMaxN; }

extern "C" uint64_t bf_abi_tag(void) { return BF_ABI_TAG; }

extern "C" size_t bf_wstream_bytes(const bf_shape* s) {
    if (!shape_ok(s)) return 0;
    return ((size_t)s->n_layers * bf::LAYER_GROUPS + bf::HEAD_GROUPS) * bf::GROUP;
}

extern "C" size_t bf_fparams_floats(const bf_shape* s) {
    if (!shape_ok(s)) return 0;
    return (size_t)s->n_layers * bf::PARAM_FLOATS + bf::GLOBAL_FLOATS;
}

extern "C" size_t bf_workspace_bytes(const bf_shape* s, int64_t n) {
    if (!shape_ok(s) || n < 1) return 0;
    const size_t slots = (size_t)((n + bf::WAVES - 1) / bf::WAVES) * bf::WAVES;
    return slots * bf::T * bf::D * sizeof(float);
}

extern "C" size_t bf_layer_stride_floats(const bf_shape* s) {
    if (!shape_ok(s)) return 0;
    return bf::PARAM_FLOATS;
}

extern "C" void bf_int8_q_max(double* s8, double* u8) {
    if (s8) *s8 = 127.0;
    if (u8) *u8 = 255.0;
}

extern "C" double bf_fp8_q_max(void) { return 8.0; }

extern "C" const char* bf_last_error(void) { return g_err; }

// Which kernel runs for these arguments (enum bf_kernel), or a negative status.
static int choose_kernel(const bf_eval_args* a) {
    if (!a) return fail(BF_ERR_ARGUMENT, "args is NULL");
    if (!board_shape_ok(&a->shape))
        return fail(BF_ERR_UNSUPPORTED,
                    "unsupported network shape: this build carries d_model=256/n_heads=8/d_ff=1024 and "
                    "d_model=512/n_heads=16/d_ff=2048, n_layers>=1, n_value in {1,3}");
    if (a->quant != BF_QUANT_INT8 && a->quant != BF_QUANT_E4M3)
        return fail(BF_ERR_ARGUMENT, "quant must be BF_QUANT_INT8 or BF_QUANT_E4M3");
    const bool have_quad = a->wstream && a->fparams, have_board = a->board_wstream && a->board_fparams;
    const bool quad_can = shape_ok(&a->shape) && have_quad;
    // the board blobs are packed for one format; the 512-wide network runs int8 only
    const bool board_can = have_board && (a->quant == BF_QUANT_INT8 || shape_ok(&a->shape));
    const bool twin_can = have_board && shape_ok(&a->shape);
    const bool octo_can = board_can;   // the same networks and formats as BOARD
    const bool duo_can = twin_can;     // the 256-wide network, both formats
    switch (a->kernel) {
    case BF_KERNEL_QUAD:
        if (!quad_can) return fail(BF_ERR_UNSUPPORTED, "the four-positions-per-workgroup kernel needs the 256-wide network and wstream/fparams");
        return BF_KERNEL_QUAD;
    case BF_KERNEL_BOARD:
        if (!board_can) return fail(BF_ERR_UNSUPPORTED, "the one-position-per-workgroup kernel needs board_wstream/board_fparams (512-wide network: the int8 format)");
        return BF_KERNEL_BOARD;
    case BF_KERNEL_TWIN:
        if (!twin_can)
            return fail(BF_ERR_UNSUPPORTED, "the two-workgroups-per-compute-unit kernel needs the 256-wide network and board_wstream/board_fparams");
        return BF_KERNEL_TWIN;
    case BF_KERNEL_OCTO:
        if (!octo_can)
            return fail(BF_ERR_UNSUPPORTED, "the eight-wavefronts-per-position kernel needs board_wstream/board_fparams (512-wide network: the int8 format)");
        return BF_KERNEL_OCTO;
    case BF_KERNEL_DUO:
        if (!duo_can)
            return fail(BF_ERR_UNSUPPORTED, "the two-positions-per-workgroup kernel needs the 256-wide network and board_wstream/board_fparams");
        return BF_KERNEL_DUO;
    case BF_KERNEL_AUTO:
        // above one position per compute unit: two positions per workgroup for int8 (2-4 % faster
        // than TWIN from 512 positions up and half its L2 traffic), TWIN for e4m3 (whose operand
        // conversions leave the two-position form short of registers)
        if (octo_can) return (twin_can && a->n > kBoardMaxN) ? (a->quant == BF_QUANT_INT8 ? BF_KERNEL_DUO : BF_KERNEL_TWIN) : BF_KERNEL_OCTO;
        if (quad_can) return BF_KERNEL_QUAD;
        return fail(BF_ERR_ARGUMENT, shape512(&a->shape)
                        ? "the 512-wide network runs on the one-position-per-workgroup kernel: int8, board_wstream/board_fparams required"
                        : "wstream/fparams must not be NULL");
    default:
        return fail(BF_ERR_ARGUMENT, "kernel must be BF_KERNEL_AUTO, BF_KERNEL_QUAD, BF_KERNEL_BOARD, BF_KERNEL_TWIN, BF_KERNEL_OCTO or BF_KERNEL_DUO");
    }
}

extern "C" int bf_kernel_choice(const bf_eval_args* args) { return choose_kernel(args); }

static int check_args(const bf_eval_args* a, bf::KArgs* k, int* kind) {
    *kind = choose_kernel(a);
    if (*kind < 0) return *kind;
    const bool board = *kind == BF_KERNEL_BOARD || *kind == BF_KERNEL_TWIN || *kind == BF_KERNEL_OCTO || *kind == BF_KERNEL_DUO;
    if (a->n < 1 || a->n > (1ll << 28)) return fail(BF_ERR_ARGUMENT, "n must be in [1, 2^28]");
    // encoder-only launch: residual stream in and out through the tap table, no board words, no heads
    const bool enc_only = a->taps && a->taps->alive;
    if (enc_only) {
        if (!a->taps->x_in || !a->taps->resid_last)
            return fail(BF_ERR_ARGUMENT, "an encoder-only launch (taps.alive) needs taps.x_in and taps.resid_last");
        if ((uintptr_t)a->taps->resid_last & 15) return fail(BF_ERR_ARGUMENT, "resid_last must be 16-byte aligned");
        if (a->leaf_index || a->leaf_count || a->active)
            return fail(BF_ERR_ARGUMENT, "an encoder-only launch takes neither active flags nor a leaf list");
    } else {
        if (!a->boards || !a->control || !a->rep) return fail(BF_ERR_ARGUMENT, "boards/control/rep must not be NULL");
        if (!a->policy || !a->promo || !a->value) return fail(BF_ERR_ARGUMENT, "policy/promo/value must not be NULL");
    }
    const uint8_t* ws = board ? a->board_wstream : a->wstream;
    const float* fp = board ? a->board_fparams : a->fparams;
    if (((uintptr_t)ws & 15) || ((uintptr_t)fp & 15))
        return fail(BF_ERR_ARGUMENT, "the parameter blobs must be 16-byte aligned");
    if (!enc_only && (((uintptr_t)a->policy & 15) || ((uintptr_t)a->promo & 7)))
        return fail(BF_ERR_ARGUMENT, "policy must be 16-byte and promo 8-byte aligned");
    if (!enc_only && (((uintptr_t)a->boards & 1) || ((uintptr_t)a->control & 1) || ((uintptr_t)a->value & 3) ||
                      ((uintptr_t)a->mask & 7) || ((uintptr_t)a->best_move & 3)))
        return fail(BF_ERR_ARGUMENT, "boards/control/value/mask/best_move must be aligned to their element size");
    if (!enc_only && a->best_move && !a->mask) return fail(BF_ERR_ARGUMENT, "best_move needs a mask");
    if ((a->leaf_index == nullptr) != (a->leaf_count == nullptr))
        return fail(BF_ERR_ARGUMENT, "leaf_index and leaf_count come together");
    if (a->leaf_index && a->active) return fail(BF_ERR_ARGUMENT, "a compacted leaf list replaces the active flags: pass one of them");
    if (((uintptr_t)a->leaf_index & 3) || ((uintptr_t)a->leaf_count & 3))
        return fail(BF_ERR_ARGUMENT, "leaf_index / leaf_count must be 4-byte aligned");
    if (a->value_mode < BF_VALUE_KING || a->value_mode > BF_VALUE_PRENORM)
        return fail(BF_ERR_ARGUMENT, "value_mode must be BF_VALUE_KING, BF_VALUE_POOLED or BF_VALUE_PRENORM");
    if (a->value_mode != BF_VALUE_KING && !board)
        return fail(BF_ERR_UNSUPPORTED, "the pooled value heads run on the BOARD, TWIN, OCTO and DUO kernels");
    if (!board && (!a->workspace || ((uintptr_t)a->workspace & 15) || a->workspace_bytes < bf_workspace_bytes(&a->shape, a->n)))
        return fail(BF_ERR_ARGUMENT, "workspace must be 16-byte aligned and hold bf_workspace_bytes(shape, n) bytes");
    memset(k, 0, sizeof(*k));
    k->boards = a->boards; k->control = a->control; k->rep = a->rep; k->mask = a->mask; k->active = a->active;
    k->leaf_index = a->leaf_index; k->leaf_count = a->leaf_count;
    k->n = (int)a->n;
    k->wstream = ws; k->fparams = fp;
    k->policy = a->policy; k->promo = a->promo; k->value = a->value; k->best = a->best_move;
    k->out_fp32 = a->out_fp32 ? 1 : 0;
    k->xpark = static_cast<float*>(a->workspace);
    k->n_layers = a->shape.n_layers; k->n_value = a->shape.n_value; k->eps = a->shape.eps;
    k->vmode = a->value_mode;
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
    if (enc_only) {   // nothing of these is read or written
        k->boards = nullptr; k->control = nullptr; k->rep = nullptr; k->mask = nullptr;
        k->policy = nullptr; k->promo = nullptr; k->value = nullptr; k->best = nullptr;
    }
    return BF_OK;
}

constexpr int DUO_ROUND = 512;   // positions the two-position kernel holds at once on 256 compute units

// Whether the current device is an MI355X-class part (gfx950), looked up once per device; the
// kernels are compiled for that architecture only.
static bool device_is_gfx950() {
    static std::atomic<unsigned long long> known{0}, good{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        fail(BF_ERR_DEVICE, "no current HIP device");
        return false;
    }
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0;
    bool ok;
    if (known.load(std::memory_order_acquire) & bit) {
        ok = good.load(std::memory_order_relaxed) & bit;
    } else {
        hipDeviceProp_t prop;
        ok = hipGetDeviceProperties(&prop, dev) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0;
        if (ok) good.fetch_or(bit, std::memory_order_relaxed);
        known.fetch_or(bit, std::memory_order_release);
    }
    if (!ok) fail(BF_ERR_DEVICE, "the current device is not a gfx950 GPU: the kernels of this library are built for MI355X only");
    return ok;
}

// the arguments of a launch over positions [first, first + count) of the caller's arrays
static bf::KArgs slice(const bf::KArgs& k, int first, int count) {
    bf::KArgs s = k;
    const size_t f = (size_t)first, logit = k.out_fp32 ? 4 : 2;
    s.n = count;
    s.boards += f * BF_TOKENS;
    s.control += f;
    s.rep += f;
    if (s.mask) s.mask += f * BF_TOKENS;
    if (s.active) s.active += f;
    s.policy = static_cast<char*>(k.policy) + f * BF_TOKENS * BF_POLICY * logit;
    s.promo = static_cast<char*>(k.promo) + f * BF_TOKENS * BF_PROMO * logit;
    s.value += f;
    if (s.best) s.best += f;
    return s;
}

static int launch(const bf_eval_args* a, const bf::KArgs& k, int kind, hipStream_t stream) {
    const int grid = (k.n + bf::WAVES - 1) / bf::WAVES;
    hipError_t e;
    if (!device_is_gfx950()) return BF_ERR_DEVICE;
    // The two-position kernel runs in rounds of 512 positions (256 compute units x 2), and a round
    // costs the same whether it is full or not.  When the library chose the kernel itself and the
    // last round would hold at most 256 positions, those go to the one-position form in a second
    // launch on the same stream, whose single round is a third shorter (640 positions: 0.33 ms
    // instead of 0.39).  Not with a leaf list (its length is on the device), taps or the profile.
    if (kind == BF_KERNEL_DUO && a->kernel == BF_KERNEL_AUTO && a->quant == BF_QUANT_INT8 && !a->taps && !k.profile &&
        !k.leaf_index && k.n > DUO_ROUND && k.n % DUO_ROUND != 0 && k.n % DUO_ROUND <= DUO_ROUND / 2) {
        const int head = k.n - k.n % DUO_ROUND;
        e = bf::launch_duo256(slice(k, 0, head), stream);
        if (e == hipSuccess) e = bf::launch_solo256(slice(k, head, k.n - head), stream);
        if (e != hipSuccess) {
            snprintf(g_err, sizeof(g_err), "kernel launch failed: %s", hipGetErrorString(e));
            return BF_ERR_LAUNCH;
        }
        return BF_OK;
    }
    if (kind == BF_KERNEL_OCTO) {
        // eight wavefronts per position: the 512-wide network and the e4m3 format on the board kernel's
        // eight-wavefront form; the 256-wide int8 network on the two-position kernel's one-position
        // form, which issues each product under the previous one's epilogue
        if (k.profile && a->shape.d_model == 512)
            e = bf::launch_octo512_prof(k, stream);
        else if (a->shape.d_model == 512)
            e = a->taps ? bf::launch_octo512_taps(k, stream) : bf::launch_octo512(k, stream);
        else if (a->quant == BF_QUANT_E4M3)
            e = k.profile ? bf::launch_octo256_fp8_prof(k, stream)
              : a->taps   ? bf::launch_octo256_fp8_taps(k, stream)
                          : bf::launch_octo256_fp8(k, stream);
        else if (k.profile)
            e = bf::launch_solo256_prof(k, stream);
        else
            e = a->taps ? bf::launch_solo256_taps(k, stream) : bf::launch_solo256(k, stream);
    } else if (kind == BF_KERNEL_DUO) {
        if (k.profile)
            e = a->quant == BF_QUANT_E4M3 ? bf::launch_duo256_fp8_prof(k, stream) : bf::launch_duo256_prof(k, stream);
        else if (a->quant == BF_QUANT_E4M3)
            e = a->taps ? bf::launch_duo256_fp8_taps(k, stream) : bf::launch_duo256_fp8(k, stream);
        else
            e = a->taps ? bf::launch_duo256_taps(k, stream) : bf::launch_duo256(k, stream);
    } else if (kind == BF_KERNEL_TWIN) {
        if (k.profile)
            e = a->quant == BF_QUANT_E4M3 ? bf::launch_twin256_fp8_prof(k, stream) : bf::launch_twin256_prof(k, stream);
        else if (a->quant == BF_QUANT_E4M3)
            e = a->taps ? bf::launch_twin256_fp8_taps(k, stream) : bf::launch_twin256_fp8(k, stream);
        else
            e = a->taps ? bf::launch_twin256_taps(k, stream) : bf::launch_twin256(k, stream);
    } else if (kind == BF_KERNEL_BOARD) {
        if (k.profile)
            e = a->shape.d_model == 512      ? bf::launch_board512_prof(k, stream)
              : a->quant == BF_QUANT_E4M3 ? bf::launch_board256_fp8_prof(k, stream)
                                          : bf::launch_board256_prof(k, stream);
        else if (a->shape.d_model == 512)
            e = a->taps ? bf::launch_board512_taps(k, stream) : bf::launch_board512(k, stream);
        else if (a->quant == BF_QUANT_E4M3)
            e = a->taps ? bf::launch_board256_fp8_taps(k, stream) : bf::launch_board256_fp8(k, stream);
        else
            e = a->taps ? bf::launch_board256_taps(k, stream) : bf::launch_board256(k, stream);
    } else if (a->quant == BF_QUANT_E4M3)
        e = k.profile ? bf::launch_prof_fp8(k, grid, stream)
          : a->taps   ? bf::launch_taps_fp8(k, grid, stream)
                      : bf::launch_prod_fp8(k, grid, stream);
    else
        e = k.profile ? bf::launch_prof(k, grid, stream)
          : a->taps   ? bf::launch_taps(k, grid, stream)
                      : bf::launch_prod(k, grid, stream);
    if (e != hipSuccess) {
        snprintf(g_err, sizeof(g_err), "kernel launch failed: %s", hipGetErrorString(e));
        return BF_ERR_LAUNCH;
    }
    return BF_OK;
}

extern "C" int bf_model_forward(const bf_eval_args* args, void* stream) {
    bf::KArgs k;
    int kind;
    const int rc = check_args(args, &k, &kind);
    if (rc) return rc;
    return launch(args, k, kind, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing ----------------------------------------------------
// The four-positions-per-workgroup kernel parks the residual stream in a workspace the caller
// lends to bf_model_forward.  For callers that cannot allocate, the same launch with the
// workspace in this file-scope device array.  Each GPU the library runs on holds its own copy
// at its own address until the process ends; `scratch` is the host-side stand-in of the symbol
// and is never passed to a kernel: host code uses the per-device address looked up below.
static __device__ __align__(256) uint8_t scratch[(size_t)BF_STATIC_MAX_N * bf::T * bf::D * sizeof(float)];

static const int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on device i, NULL until looked up

// The address of this device's copy of `scratch`, looked up once per device with that device
// current (the caller's current device is the one the launch goes to).
static int scratch_address(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(BF_ERR_DEVICE, "no current HIP device (or its ordinal is 64 or more)");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            snprintf(g_err, sizeof(g_err), "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return BF_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return BF_OK;
}

extern "C" int bf_model_forward_static(const bf_eval_args* args, void* stream) {
    if (!args) return fail(BF_ERR_ARGUMENT, "args is NULL");
    if (args->kernel != BF_KERNEL_AUTO && args->kernel != BF_KERNEL_QUAD)
        return fail(BF_ERR_ARGUMENT, "bf_model_forward_static runs the four-positions-per-workgroup kernel: kernel must be BF_KERNEL_QUAD "
                                     "or BF_KERNEL_AUTO (the other kernels need no workspace: call bf_model_forward)");
    if (args->n > BF_STATIC_MAX_N) {
        snprintf(g_err, sizeof(g_err), "n = %lld exceeds BF_STATIC_MAX_N = %d positions, the size of the library's static workspace",
                 (long long)args->n, BF_STATIC_MAX_N);
        return BF_ERR_ARGUMENT;
    }
    // the argument checks come first (they touch no device); the placeholder only has to pass them
    bf_eval_args a = *args;
    a.kernel = BF_KERNEL_QUAD;
    a.workspace = reinterpret_cast<void*>(uintptr_t(256));
    a.workspace_bytes = sizeof(scratch);
    bf::KArgs k;
    int kind;
    const int rc = check_args(&a, &k, &kind);
    if (rc) return rc;
    void* ws = nullptr;
    const int rc0 = scratch_address(&ws);
    if (rc0) return rc0;
    k.xpark = static_cast<float*>(ws);
    return launch(&a, k, kind, (hipStream_t)stream);
}

extern "C" int bf_profile_phases(const bf_eval_args* args, void* stream, uint64_t* cycles) {
    bf::KArgs k;
    int kind;
    const int rc = check_args(args, &k, &kind);
    if (rc) return rc;
    if (args->taps) return fail(BF_ERR_ARGUMENT, "the phase profile runs without taps");
    if (!cycles) return fail(BF_ERR_ARGUMENT, "cycles must not be NULL");
    k.profile = reinterpret_cast<unsigned long long*>(cycles);
    return launch(args, k, kind, (hipStream_t)stream);
}

extern "C" int bf_profile_phase_count(void) { return bf::N_PHASES; }

extern "C" const char* bf_profile_phase_name(int i) {
    static const char* names[bf::N_PHASES] = {"embed", "ln1_quant", "qkv_gemm_epilogue", "attention",
                                              "oquant_outproj", "ln2_quant", "ffn1", "ffn2", "heads",
                                              "store", "sync_wait", "total"};
    return (i >= 0 && i < bf::N_PHASES) ? names[i] : "";
}

extern "C" double bf_time_kernel_ms(const bf_eval_args* args, void* stream, int warmup, int iters) {
    bf::KArgs k;
    int kind;
    int rc = check_args(args, &k, &kind);
    if (rc) return rc;
    if (iters < 1 || warmup < 0) return fail(BF_ERR_ARGUMENT, "iters must be >= 1 and warmup >= 0");
    hipStream_t s = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BF_ERR_LAUNCH, "hipEventCreate failed");
    }
    for (int i = 0; i < warmup && !rc; i++) rc = launch(args, k, kind, s);
    (void)hipEventRecord(e0, s);
    for (int i = 0; i < iters && !rc; i++) rc = launch(args, k, kind, s);
    (void)hipEventRecord(e1, s);
    const hipError_t e = hipEventSynchronize(e1);
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    if (e != hipSuccess) return fail(BF_ERR_LAUNCH, hipGetErrorString(e));
    return (double)ms / iters;
}
