// ckpt_tool.cpp
//
// The C++ half of the cross-language optimizer-state tests (tests/test_gpu_loop.py): a small model in the
// reference's pool layout, stepped through the reference's call sequence (clip_grad_norm_, step), with the
// optimizer state saved to or loaded from a file that the Python AdamWOptimizer also reads and writes.
//
//   ckpt_tool save <dir> <k>        seeded weights, steps 1..k, then <dir>/opt.state and the weights
//                                   (<dir>/w16.bin, <dir>/w32.bin: the model's to save, not the optimizer's)
//   ckpt_tool load <dir> <k> <j>    weights and state from <dir> (must be at step k), steps k+1..k+j, then
//                                   <dir>/out_{w16,w32,master,m16,v16,m32,v32}.bin
// Gradients of step s: FP16 pool from seed 5000+2s, FP32 pool (norm gradients + workspace tail) from 5001+2s.
// Exit code 0 = done, 3 = the state file was refused, anything else = failure.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "training/optimizer.h"

namespace {

struct Config {      // a Qwen3-shaped model whose every tensor is a multiple of 128 elements
    int vocab_size = 512, hidden_size = 128, intermediate_size = 256, num_hidden_layers = 2, head_dim = 128;
    int q_dim = 256, kv_dim = 128;
};
struct Weights { half* fp16_pool = nullptr; float* fp32_pool = nullptr; size_t fp16_pool_elems = 0, fp32_pool_elems = 0; };
struct Model { Config config; Weights weights; };
struct Grads { half* half_pool = nullptr; float* float_pool = nullptr; size_t half_pool_bytes = 0, float_pool_bytes = 0; };

constexpr size_t kTail = 148;            // workspace floats behind the norm gradients
constexpr float kLr = 1e-3f, kMaxNorm = 0.5f, kGradStd = 5e-3f;

bool write_file(const std::string& path, const void* dev, size_t bytes) {
    std::vector<char> h(bytes);
    HIP_CHECK(hipMemcpy(h.data(), dev, bytes, hipMemcpyDeviceToHost));
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) return false;
    const bool ok = fwrite(h.data(), 1, bytes, f) == bytes;
    return fclose(f) == 0 && ok;
}

bool read_file(const std::string& path, void* dev, size_t bytes) {
    std::vector<char> h(bytes);
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return false;
    const bool ok = fread(h.data(), 1, bytes, f) == bytes;
    fclose(f);
    if (ok) HIP_CHECK(hipMemcpy(dev, h.data(), bytes, hipMemcpyHostToDevice));
    return ok;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc < 4) { fprintf(stderr, "usage: ckpt_tool save <dir> <k> | load <dir> <k> <j>\n"); return 2; }
    const std::string mode = argv[1], dir = argv[2];
    const int k = atoi(argv[3]), j = argc > 4 ? atoi(argv[4]) : 0;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) { fprintf(stderr, "no GPU\n"); return 2; }

    Model model;
    const Config& c = model.config;
    const size_t H = c.hidden_size;
    const size_t n16 = (2 * (size_t)c.q_dim * H + 2 * (size_t)c.kv_dim * H + 3 * (size_t)c.intermediate_size * H) *
                           c.num_hidden_layers + (size_t)c.vocab_size * H;
    const size_t n32 = (2 * H + 2 * c.head_dim) * c.num_hidden_layers + H;
    model.weights.fp16_pool_elems = n16;
    model.weights.fp32_pool_elems = n32;
    HIP_CHECK(hipMalloc((void**)&model.weights.fp16_pool, n16 * 2));
    HIP_CHECK(hipMalloc((void**)&model.weights.fp32_pool, n32 * 4));
    Grads grads;
    grads.half_pool_bytes = n16 * 2;
    grads.float_pool_bytes = (n32 + kTail) * 4;
    HIP_CHECK(hipMalloc((void**)&grads.half_pool, grads.half_pool_bytes));
    HIP_CHECK(hipMalloc((void**)&grads.float_pool, grads.float_pool_bytes));

    int first = 1, last = k;
    if (mode == "save") {
        RLX_CHECK(rlx_fill_f16((uint16_t*)model.weights.fp16_pool, n16, 71, 0, 0.0f, 0.02f, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(model.weights.fp32_pool, n32, 72, 0, 1.0f, 0.05f, 0, 0, 0, nullptr));
    } else if (mode == "load") {
        if (!read_file(dir + "/w16.bin", model.weights.fp16_pool, n16 * 2) ||
            !read_file(dir + "/w32.bin", model.weights.fp32_pool, n32 * 4)) { fprintf(stderr, "cannot read the weights\n"); return 4; }
        first = k + 1;
        last = k + j;
    } else {
        return 2;
    }
    HIP_CHECK(hipDeviceSynchronize());

    AdamWOptimizer optimizer(&model, kLr);           // master copy from the weights as they are now
    if (mode == "load") {
        if (!optimizer.load_state(dir + "/opt.state")) return 3;
        if (optimizer.get_step() != k) { fprintf(stderr, "state is at step %d, expected %d\n", optimizer.get_step(), k); return 5; }
    }
    for (int s = first; s <= last; s++) {
        RLX_CHECK(rlx_fill_f16((uint16_t*)grads.half_pool, n16, 5000 + 2 * s, 0, 0.0f, kGradStd, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(grads.float_pool, n32 + kTail, 5001 + 2 * s, 0, 0.0f, kGradStd, 0, 0, 0, nullptr));
        const float norm = clip_grad_norm_(optimizer, &grads, kMaxNorm);
        optimizer.step(&grads);
        printf("step %d norm %.9g\n", s, norm);
    }
    HIP_CHECK(hipDeviceSynchronize());

    bool ok = true;
    if (mode == "save") {
        ok = optimizer.save_state(dir + "/opt.state") && write_file(dir + "/w16.bin", model.weights.fp16_pool, n16 * 2) &&
             write_file(dir + "/w32.bin", model.weights.fp32_pool, n32 * 4);
    } else {
        ok = write_file(dir + "/out_w16.bin", model.weights.fp16_pool, n16 * 2) &&
             write_file(dir + "/out_w32.bin", model.weights.fp32_pool, n32 * 4) &&
             write_file(dir + "/out_master.bin", optimizer.fp16_master(), n16 * 4) &&
             write_file(dir + "/out_m16.bin", optimizer.fp16_m(), n16 * 4) &&
             write_file(dir + "/out_v16.bin", optimizer.fp16_v(), n16 * 4) &&
             write_file(dir + "/out_m32.bin", optimizer.fp32_m(), n32 * 4) &&
             write_file(dir + "/out_v32.bin", optimizer.fp32_v(), n32 * 4);
    }
    (void)hipFree(model.weights.fp16_pool); (void)hipFree(model.weights.fp32_pool);
    (void)hipFree(grads.half_pool); (void)hipFree(grads.float_pool);
    return ok ? 0 : 6;
}
