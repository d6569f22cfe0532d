// A host program that uses the evaluator through its C-ABI alone (include/brokefish_hip.h and the
// HIP runtime: no PyTorch, no Python): it reads the packed parameter blobs and a batch of positions
// from files, runs move generation, the evaluator with the legal-move AND and the edge expansion
// on a stream of its own, and writes the outputs to files.  tests/test_c_driver_gpu.py feeds it
// what the Python packer produced and compares the files with the Python binding's results, bit
// for bit.  Usage: c_driver <dir> <n> <n_value>; files in <dir>: wstream.bin, fparams.bin,
// boards.bin, control.bin, rep.bin -> policy.bin, promo.bin, value.bin, best.bin, mask.bin,
// edge_move.bin, edge_prior.bin, n_edges.bin
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "brokefish_hip.h"

#define HIP_OK(x)                                                                        \
    do {                                                                                 \
        const hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                          \
            fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));               \
            return 2;                                                                    \
        }                                                                                \
    } while (0)
#define BF_OK_OR_DIE(x)                                                                  \
    do {                                                                                 \
        const int rc_ = (x);                                                             \
        if (rc_ != BF_OK) {                                                              \
            fprintf(stderr, "%s failed (%d): %s\n", #x, rc_, bf_last_error());           \
            return 3;                                                                    \
        }                                                                                \
    } while (0)

static std::vector<char> read_file(const std::string& path) {
    std::vector<char> v;
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return v;
    fseek(f, 0, SEEK_END);
    v.resize((size_t)ftell(f));
    fseek(f, 0, SEEK_SET);
    if (fread(v.data(), 1, v.size(), f) != v.size()) v.clear();
    fclose(f);
    return v;
}
static bool write_file(const std::string& path, const void* p, size_t bytes) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) return false;
    const bool ok = fwrite(p, 1, bytes, f) == bytes;
    fclose(f);
    return ok;
}

int main(int argc, char** argv) {
    if (argc != 4) {
        fprintf(stderr, "usage: %s <dir> <n> <n_value>\n", argv[0]);
        return 1;
    }
    const std::string dir = std::string(argv[1]) + "/";
    const int64_t n = atoll(argv[2]);
    const bf_shape shape = {256, 8, 8, 1024, atoi(argv[3]), 1e-5f};
    if (bf_abi_tag() != BF_ABI_TAG) {
        fprintf(stderr, "library and header disagree about the interface\n");
        return 1;
    }
    const std::vector<char> ws = read_file(dir + "wstream.bin"), fp = read_file(dir + "fparams.bin");
    const std::vector<char> boards = read_file(dir + "boards.bin"), control = read_file(dir + "control.bin"),
                            rep = read_file(dir + "rep.bin");
    if (ws.size() != bf_board_wstream_bytes(&shape) || fp.size() != 4 * bf_board_fparams_floats(&shape)) {
        fprintf(stderr, "the blobs are not those of this shape (%zu, %zu bytes)\n", ws.size(), fp.size());
        return 1;
    }
    if (boards.size() != (size_t)n * 64 || control.size() != (size_t)n * 2 || rep.size() != (size_t)n) {
        fprintf(stderr, "the position files do not hold %lld positions\n", (long long)n);
        return 1;
    }
    const int E = 96;
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    void *d_ws, *d_fp, *d_boards, *d_control, *d_rep, *d_mask, *d_check, *d_policy, *d_promo, *d_value, *d_best;
    void *d_move, *d_prior, *d_nedges;
    HIP_OK(hipMalloc(&d_ws, ws.size()));
    HIP_OK(hipMalloc(&d_fp, fp.size()));
    HIP_OK(hipMalloc(&d_boards, boards.size()));
    HIP_OK(hipMalloc(&d_control, control.size()));
    HIP_OK(hipMalloc(&d_rep, rep.size()));
    HIP_OK(hipMalloc(&d_mask, (size_t)n * 32 * 8));
    HIP_OK(hipMalloc(&d_check, (size_t)n));
    HIP_OK(hipMalloc(&d_policy, (size_t)n * 32 * 64 * 2));
    HIP_OK(hipMalloc(&d_promo, (size_t)n * 32 * 4 * 2));
    HIP_OK(hipMalloc(&d_value, (size_t)n * 4));
    HIP_OK(hipMalloc(&d_best, (size_t)n * 4));
    HIP_OK(hipMalloc(&d_move, (size_t)n * E * 2));
    HIP_OK(hipMalloc(&d_prior, (size_t)n * E * 2));
    HIP_OK(hipMalloc(&d_nedges, (size_t)n * 4));
    HIP_OK(hipMemcpyAsync(d_ws, ws.data(), ws.size(), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_fp, fp.data(), fp.size(), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_boards, boards.data(), boards.size(), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_control, control.data(), control.size(), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_rep, rep.data(), rep.size(), hipMemcpyHostToDevice, stream));

    // legal-move words, then the evaluator with the mask ANDed in, then the edges: three launches
    // on one stream, nothing through the host in between
    BF_OK_OR_DIE(bf_movegen((const uint16_t*)d_boards, (const int16_t*)d_control, n, (uint64_t*)d_mask, (uint8_t*)d_check, stream));
    bf_eval_args a = {};
    a.boards = (const uint16_t*)d_boards;
    a.control = (const int16_t*)d_control;
    a.rep = (const uint8_t*)d_rep;
    a.mask = (const uint64_t*)d_mask;
    a.n = n;
    a.shape = shape;
    a.board_wstream = (const uint8_t*)d_ws;
    a.board_fparams = (const float*)d_fp;
    a.policy = d_policy;
    a.promo = d_promo;
    a.value = (float*)d_value;
    a.best_move = (int32_t*)d_best;
    a.quant = BF_QUANT_INT8;
    a.kernel = BF_KERNEL_AUTO;
    a.value_mode = BF_VALUE_KING;
    BF_OK_OR_DIE(bf_model_forward(&a, stream));
    bf_expand_args x = {};
    x.policy = d_policy;
    x.promo = d_promo;
    x.value = (const float*)d_value;
    x.mask = (const uint64_t*)d_mask;
    x.boards = (const uint16_t*)d_boards;
    x.control = (const int16_t*)d_control;
    x.n = n;
    x.max_edges = E;
    x.edge_move = (int16_t*)d_move;
    x.edge_prior = d_prior;
    x.n_edges = (int32_t*)d_nedges;
    BF_OK_OR_DIE(bf_expand(&x, stream));
    HIP_OK(hipStreamSynchronize(stream));

    struct Out { const char* name; void* dev; size_t bytes; };
    const Out outs[] = {{"policy.bin", d_policy, (size_t)n * 32 * 64 * 2}, {"promo.bin", d_promo, (size_t)n * 32 * 4 * 2},
                        {"value.bin", d_value, (size_t)n * 4}, {"best.bin", d_best, (size_t)n * 4},
                        {"mask.bin", d_mask, (size_t)n * 32 * 8}, {"edge_move.bin", d_move, (size_t)n * E * 2},
                        {"edge_prior.bin", d_prior, (size_t)n * E * 2}, {"n_edges.bin", d_nedges, (size_t)n * 4}};
    for (const Out& o : outs) {
        std::vector<char> h(o.bytes);
        HIP_OK(hipMemcpy(h.data(), o.dev, o.bytes, hipMemcpyDeviceToHost));
        if (!write_file(dir + o.name, h.data(), o.bytes)) {
            fprintf(stderr, "cannot write %s\n", o.name);
            return 1;
        }
    }
    printf("c_driver: %lld positions, kernel %d\n", (long long)n, bf_kernel_choice(&a));
    return 0;
}
