/* Plain C99 client of the evaluator's C-ABI: proves that include/brokefish_hip.h is valid C,
 * that every entry point links, and that argument errors come back as statuses (no device is
 * touched: every call below fails its argument check first). Built and run by tests/test_host.py. */
#include <stdio.h>
#include <string.h>

#include "brokefish_hip.h"

int main(void) {
    bf_shape shape;
    bf_eval_args args;
    bf_expand_args ex;
    double s8 = 0.0, u8 = 0.0;

    memset(&shape, 0, sizeof shape);
    shape.d_model = 256; shape.n_layers = 8; shape.n_heads = 8; shape.d_ff = 1024; shape.n_value = 1; shape.eps = 1e-5f;
    if (bf_wstream_bytes(&shape) == 0 || bf_fparams_floats(&shape) == 0 || bf_workspace_bytes(&shape, 4096) == 0) return 1;
    if (bf_board_wstream_bytes(&shape) == 0 || bf_board_fparams_floats(&shape) == 0 || bf_layer_stride_floats(&shape) == 0) return 2;
    if (bf_board_max_n() < 1) return 3;
    bf_int8_q_max(&s8, &u8);
    if (s8 != 127.0 || u8 != 255.0 || bf_fp8_q_max() != 8.0) return 4;

    memset(&args, 0, sizeof args);
    args.shape = shape;
    args.n = 16;
    if (bf_model_forward(&args, NULL) != BF_ERR_ARGUMENT || strlen(bf_last_error()) == 0) return 5;
    if (bf_model_forward(NULL, NULL) != BF_ERR_ARGUMENT) return 6;
    if (bf_model_forward_static(&args, NULL) >= 0 || bf_model_forward_static(NULL, NULL) != BF_ERR_ARGUMENT) return 15;   /* no parameter blobs */
    args.n = BF_STATIC_MAX_N + 1;
    if (bf_model_forward_static(&args, NULL) != BF_ERR_ARGUMENT || !strstr(bf_last_error(), "BF_STATIC_MAX_N")) return 16;
    args.n = 16;
    if (bf_kernel_choice(&args) >= 0) return 7;                 /* no parameter blobs */
    if (bf_time_kernel_ms(&args, NULL, 1, 1) >= 0.0) return 8;
    if (bf_profile_phases(&args, NULL, NULL) >= 0) return 9;
    if (bf_profile_phase_count() < 1 || strlen(bf_profile_phase_name(0)) == 0) return 10;
    shape.d_model = 384;
    args.shape = shape;
    if (bf_model_forward(&args, NULL) != BF_ERR_UNSUPPORTED) return 11;

    memset(&ex, 0, sizeof ex);
    if (bf_expand(&ex, NULL) != BF_ERR_ARGUMENT || bf_expand(NULL, NULL) != BF_ERR_ARGUMENT) return 12;
    if (bf_movegen(NULL, NULL, 4, NULL, NULL, NULL) != BF_ERR_ARGUMENT) return 13;
    if (bf_compact_leaves(NULL, 4, NULL, NULL, NULL) != BF_ERR_ARGUMENT) return 17;
    if (bf_mfma_rate(BF_QUANT_INT8, NULL, 10, 1, NULL) >= 0.0) return 14;
    if (bf_stream_rate(NULL, 32768, 4, 1, NULL, NULL) >= 0.0) return 18;
    if (bf_abi_tag() != BF_ABI_TAG || (bf_abi_tag() >> 32) != BF_ABI_VERSION) return 19;    /* this client and the library agree */
    if (bf_quant_probe(BF_PROBE_S8, NULL, 1.0f, 4, NULL, NULL) != BF_ERR_ARGUMENT) return 20;
    printf("abi ok: %s\n", bf_last_error());
    return 0;
}
