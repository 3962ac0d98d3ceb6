// C++ host program in the shape of the reference's transformer_inference_part.cpp: the same command line
// (batch_size num_layers seq_len head_num size_per_head, transformer_inference_part.cpp:32-36), byte vocabulary
// of 256 (:38), weights drawn N(0, 0.02) with gains 1 and biases 0 (transformer.cpp:98-136), causal attention,
// then ONE forward pass (:190-256): embedding + position, num_layers pre-LN layers, tied logits, cross-entropy
// loss, printed like the reference (:255).  Inputs are synthetic bytes (the reference reads files xs0 / ys0,
// which are not part of its repository).  The program checks the loss against a double-precision recomputation
// from the device logits and against ln(256), the loss of a model that knows nothing.  Exit code 0 = passed.
//   usage: transformer_inference [batch_size num_layers seq_len head_num size_per_head [bf16|f32]]
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "device_ops.h"

#define HIP_OK(call)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            return 2;                                                                     \
        }                                                                                 \
    } while (0)

static std::mt19937_64 g_rng(20240611);

static float* normal_on_device(size_t n, float std_dev, float mean) {
    std::vector<float> h(n);
    std::normal_distribution<float> dist(mean, std_dev);
    for (auto& x : h) x = std_dev > 0 ? dist(g_rng) : mean;
    float* d = nullptr;
    if (hipMalloc((void**)&d, n * sizeof(float)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), n * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}

static void* bf16_copy(const float* d_src, size_t n) {
    void* d = nullptr;
    if (hipMalloc(&d, n * 2) != hipSuccess) return nullptr;
    if (sfb_cast_f32_bf16(nullptr, d, d_src, n) != SFB_OK) return nullptr;
    return d;
}

int main(int argc, char** argv) {
    const int batch_size = argc > 1 ? std::atoi(argv[1]) : 2;
    const int num_layers = argc > 2 ? std::atoi(argv[2]) : 2;
    const int seq_len = argc > 3 ? std::atoi(argv[3]) : 1024;
    const int head_num = argc > 4 ? std::atoi(argv[4]) : 8;
    const int size_per_head = argc > 5 ? std::atoi(argv[5]) : 64;
    const int dtype = (argc > 6 && !std::strcmp(argv[6], "f32")) ? SFB_F32 : SFB_BF16;
    const int vocab_size = 256, blk = 64;
    const int state = head_num * size_per_head, ffn = state * 4;
    const size_t m = (size_t)batch_size * seq_len;
    if (batch_size < 1 || num_layers < 0 || seq_len % blk || head_num < 1 || size_per_head != 64) {
        std::fprintf(stderr, "seq_len must be a multiple of %d and size_per_head 64\n", blk);
        return 1;
    }
    const int nb = seq_len / blk;

    // descriptors: causal layout with triangular diagonal blocks (no_fusion_test.cu:47-62, 124-143)
    std::vector<uint32_t> layout((size_t)nb * nb);
    if (sfb_layout_full(layout.data(), nb, 1) != SFB_OK) return 1;
    const uint32_t blocks = sfb_count_blocks(layout.data(), nb);
    std::vector<sfb_uint2> nt(blocks), nn(nb + blocks);
    uint32_t nn_max = 0;
    sfb_build_nt_lut(nt.data(), layout.data(), nb);
    sfb_build_nn_lut(nn.data(), nt.data(), blocks, nb, &nn_max);
    std::vector<uint8_t> keep((size_t)blocks * blk * blk);
    sfb_element_mask(keep.data(), nt.data(), blocks, blk, 1, 0);
    std::vector<uint64_t> mask((size_t)blocks * blk);
    sfb_pack_mask(mask.data(), keep.data(), blocks, blk);
    sfb_uint2* d_nn = nullptr;
    uint64_t* d_mask = nullptr;
    HIP_OK(hipMalloc((void**)&d_nn, nn.size() * sizeof(sfb_uint2)));
    HIP_OK(hipMemcpy(d_nn, nn.data(), nn.size() * sizeof(sfb_uint2), hipMemcpyHostToDevice));
    HIP_OK(hipMalloc((void**)&d_mask, mask.size() * 8));
    HIP_OK(hipMemcpy(d_mask, mask.data(), mask.size() * 8, hipMemcpyHostToDevice));
    // rows much longer than a work-group's share of the launch are split into chunks so that the launch is balanced
    const uint32_t max_blocks = sfb_suggest_max_blocks(nn.data(), nb, (uint32_t)(batch_size * head_num));
    uint32_t n_items = 0, n_heavy = 0, n_slots = 0, n_parts = 0;
    sfb_build_schedule(nullptr, &n_items, &n_heavy, &n_slots, &n_parts, nn.data(), nb, max_blocks);
    std::vector<sfb_work_item> items(n_items);
    sfb_build_schedule(items.data(), &n_items, &n_heavy, &n_slots, &n_parts, nn.data(), nb, max_blocks);
    sfb_work_item* d_items = nullptr;
    HIP_OK(hipMalloc((void**)&d_items, items.size() * sizeof(sfb_work_item)));
    HIP_OK(hipMemcpy(d_items, items.data(), items.size() * sizeof(sfb_work_item), hipMemcpyHostToDevice));
    size_t attn_ws_bytes = sfb_schedule_workspace_bytes(n_slots, n_parts, batch_size, head_num, blk, size_per_head);
    if (attn_ws_bytes < 256) attn_ws_bytes = 256;
    void* d_attn_ws = nullptr;
    HIP_OK(hipMalloc(&d_attn_ws, attn_ws_bytes));
    HIP_OK(hipMemset(d_attn_ws, 0, attn_ws_bytes));

    // weights (transformer.cpp:98-136)
    std::vector<sfb_layer_weights> layers(num_layers);
    for (auto& l : layers) {
        const float* mats[6];
        const size_t sizes[6] = {(size_t)state * state, (size_t)state * state, (size_t)state * state,
                                 (size_t)state * state, (size_t)state * ffn,   (size_t)ffn * state};
        for (int i = 0; i < 6; ++i) {
            float* w = normal_on_device(sizes[i], 0.02f, 0.f);
            if (!w) return 2;
            mats[i] = w;
            if (dtype == SFB_BF16) {
                mats[i] = (const float*)bf16_copy(w, sizes[i]);
                HIP_OK(hipDeviceSynchronize());
                HIP_OK(hipFree(w));
            }
        }
        l.wq = mats[0]; l.wk = mats[1]; l.wv = mats[2]; l.wo = mats[3]; l.w1 = mats[4]; l.w2 = mats[5];
        l.bq = normal_on_device(state, 0, 0); l.bk = normal_on_device(state, 0, 0);
        l.bv = normal_on_device(state, 0, 0); l.bo = normal_on_device(state, 0, 0);
        l.b1 = normal_on_device(ffn, 0, 0);   l.b2 = normal_on_device(state, 0, 0);
        l.ln1_g = normal_on_device(state, 0, 1); l.ln1_b = normal_on_device(state, 0, 0);
        l.ln2_g = normal_on_device(state, 0, 1); l.ln2_b = normal_on_device(state, 0, 0);
        // Q, K and V as one product: [Wq | Wk | Wv] and [bq | bk | bv] side by side
        void* wqkv = nullptr;
        float* bqkv = nullptr;
        HIP_OK(hipMalloc(&wqkv, (size_t)3 * state * state * (dtype == SFB_BF16 ? 2 : 4)));
        HIP_OK(hipMalloc((void**)&bqkv, (size_t)3 * state * sizeof(float)));
        if (sfb_pack_qkv(nullptr, wqkv, bqkv, &l, dtype, (uint32_t)state) != SFB_OK) return 2;
        HIP_OK(hipDeviceSynchronize());
        l.wqkv = wqkv;
        l.bqkv = bqkv;
    }
    sfb_model_weights w;
    w.tok_embed = normal_on_device((size_t)vocab_size * state, 0.02f, 0.f);
    w.pos_embed = normal_on_device((size_t)seq_len * state, 0.02f, 0.f);
    w.tok_embed_bf16 = dtype == SFB_BF16 ? bf16_copy(w.tok_embed, (size_t)vocab_size * state) : nullptr;
    w.layers = layers.data();
    w.n_layers = (uint32_t)num_layers;

    // synthetic bytes in place of xs0 / ys0 (next-byte targets)
    std::vector<int> xs(m), ys(m);
    for (size_t i = 0; i < m; ++i) xs[i] = (int)(g_rng() % vocab_size);
    for (size_t i = 0; i < m; ++i) ys[i] = (i + 1) % seq_len ? xs[i + 1 < m ? i + 1 : i] : (int)(g_rng() % vocab_size);
    int *d_xs = nullptr, *d_ys = nullptr;
    HIP_OK(hipMalloc((void**)&d_xs, m * sizeof(int)));
    HIP_OK(hipMalloc((void**)&d_ys, m * sizeof(int)));
    HIP_OK(hipMemcpy(d_xs, xs.data(), m * sizeof(int), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_ys, ys.data(), m * sizeof(int), hipMemcpyHostToDevice));

    const size_t ws_bytes = sfb_model_workspace_bytes(batch_size, seq_len, head_num, size_per_head, ffn, vocab_size, dtype);
    void* d_ws = nullptr;
    float *d_loss = nullptr, *d_logits = nullptr;
    HIP_OK(hipMalloc((void**)&d_logits, m * vocab_size * sizeof(float)));
    HIP_OK(hipMalloc(&d_ws, ws_bytes));
    HIP_OK(hipMalloc((void**)&d_loss, sizeof(float)));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    float loss = 0;
    double ms = 0;
    for (int iter = 0; iter < 3; ++iter) {   // the first pass also pays for library initialisation
        HIP_OK(hipStreamSynchronize(stream));
        const auto t0 = std::chrono::steady_clock::now();
        const int rc = sfb_model_forward(stream, d_loss, d_logits, nullptr, d_xs, d_ys, &w, dtype, 1, d_nn, d_mask, nullptr,
                                         d_items, n_items, n_heavy, n_slots, n_parts, d_attn_ws, attn_ws_bytes, blk,
                                         blocks, batch_size, nb, head_num, size_per_head, ffn, vocab_size, d_ws,
                                         ws_bytes);
        if (rc != SFB_OK) {
            std::fprintf(stderr, "sfb_model_forward: %s\n", sfb_status_string(rc));
            return 1;
        }
        HIP_OK(hipStreamSynchronize(stream));
        ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        HIP_OK(hipMemcpy(&loss, d_loss, sizeof(float), hipMemcpyDeviceToHost));
    }
    std::printf("batch %d layers %d seq_len %d heads %d size_per_head %d %s: forward %.3f ms\n", batch_size, num_layers,
                seq_len, head_num, size_per_head, dtype == SFB_BF16 ? "bf16" : "f32", ms);
    std::printf("loss: %.10f \n", loss);
    // the loss recomputed on the host in double precision from the logits the device produced
    std::vector<float> logits(m * vocab_size);
    HIP_OK(hipMemcpy(logits.data(), d_logits, logits.size() * sizeof(float), hipMemcpyDeviceToHost));
    double host_loss = 0;
    for (size_t r = 0; r < m; ++r) {
        const float* row = logits.data() + r * vocab_size;
        double mx = row[0], sum = 0;
        for (int j = 1; j < vocab_size; ++j) mx = std::fmax(mx, row[j]);
        for (int j = 0; j < vocab_size; ++j) sum += std::exp(row[j] - mx);
        host_loss += mx + std::log(sum) - row[ys[r]];
    }
    host_loss /= (double)m;
    // a freshly initialised model knows nothing: its loss is ln(256) plus half the variance of its logits
    const double uninformed = std::log((double)vocab_size);
    const bool ok = std::isfinite(loss) && std::fabs(loss - host_loss) <= 1e-4 * host_loss &&
                    loss > 0.98 * uninformed && loss < 1.25 * uninformed;
    std::printf("loss recomputed on the host from the device logits: %.10f; ln 256 = %.4f\n", host_loss, uninformed);
    std::printf(ok ? "PASSED\n" : "FAILED\n");
    return ok ? 0 : 1;
}
