// Host-side sanitizer run of the C ABI (AddressSanitizer + UndefinedBehaviorSanitizer on the host code only): every
// entry point that can run without a GPU, the error paths of those that cannot, and the clean-up of a model whose
// construction fails half-way.  Built and run by tests/test_host_sanitize.py; prints "ok" and returns 0.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/llama2_hip.h"
#include "../../include/llama2_hip_bench.h"

#define REQUIRE(cond)                                                     \
    do {                                                                  \
        if (!(cond)) {                                                    \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, #cond);    \
            return 1;                                                     \
        }                                                                 \
    } while (0)

int main(int argc, char **argv) {
    REQUIRE(argc == 2); // path of the tokenizer file
    // presets and sizes (src/constants.rs:7-41)
    l2_dims d{};
    REQUIRE(l2_preset("7B", 128, &d) == L2_OK && d.dim == 4096 && d.n_layers == 32);
    REQUIRE(l2_preset("70B", 64, &d) == L2_OK && d.n_kv_heads == 8);
    REQUIRE(l2_preset("9B", 128, &d) != L2_OK);
    REQUIRE(strlen(l2_last_error()) > 0);
    REQUIRE(l2_preset(nullptr, 128, &d) != L2_OK);

    // a small synthetic checkpoint, then a model on it: without a device the construction fails after the host
    // side of it has run, and must release what it holds
    l2_dims t{};
    t.dim = 256, t.hidden_dim = 384, t.n_layers = 2, t.n_heads = 2, t.n_kv_heads = 1, t.vocab_size = 96, t.seq_len = 32,
    t.group_size = 128;
    const size_t nb = l2_weights_bytes(&t);
    REQUIRE(nb > 0);
    std::vector<char> img(nb);
    REQUIRE(l2_synth_image(&t, 3, img.data(), nb) == L2_OK);
    REQUIRE(l2_synth_image(&t, 3, img.data(), nb - 1) != L2_OK);
    std::vector<char> img2(nb);
    REQUIRE(l2_synth_image(&t, 3, img2.data(), nb) == L2_OK);
    REQUIRE(memcmp(img.data(), img2.data(), nb) == 0); // seeded, thread-count independent
    l2_model *m = nullptr;
    const int have_gpu = l2_device_count() > 0;
    int rc = l2_model_from_image(img.data(), nb, &t, 0, &m);
    if (!have_gpu) REQUIRE(rc != L2_OK && m == nullptr);
    REQUIRE(l2_model_from_image(img.data(), nb - 4, &t, 0, &m) != L2_OK);
    REQUIRE(l2_model_from_image(nullptr, nb, &t, 0, &m) != L2_OK);
    REQUIRE(l2_model_open("/nonexistent/file.bin", &t, 0, &m) != L2_OK);
    if (rc == L2_OK) l2_model_close(m);
    m = nullptr;

    // null handles everywhere
    l2_state *s = nullptr;
    int32_t tok = 1, pos = 0, nxt = 0;
    float f = 0.f;
    REQUIRE(l2_state_new(nullptr, &s) != L2_OK);
    REQUIRE(l2_forward(nullptr, nullptr, &tok, &pos, 1, nullptr) != L2_OK);
    REQUIRE(l2_prefill_chunks(nullptr, nullptr, &tok, 1, 0, 1) != L2_OK);
    REQUIRE(l2_decode_greedy(nullptr, nullptr, tok, pos, &nxt) != L2_OK);
    REQUIRE(l2_model_qmatvec(nullptr, 0, 0, &f, 1, &f) != L2_OK);
    REQUIRE(l2_model_classifier(nullptr, &f, &f) != L2_OK);
    REQUIRE(l2_qlinear_matvec(nullptr, &f, 1, &f) != L2_OK);
    REQUIRE(l2_qlinear_matvec_device(nullptr, &f, 1, &f, nullptr) != L2_OK);
    REQUIRE(l2_model_set_prefill_mode(nullptr, 0) != L2_OK);
    REQUIRE(l2_model_max_seq(nullptr) == 0);
    l2_model_close(nullptr);
    l2_state_free(nullptr);
    l2_qlinear_free(nullptr);
    l2_tokenizer_free(nullptr);
    l2_random_free(nullptr);

    // the q4 launcher's planning and argument building for every decode launch of the three presets (no device,
    // nothing launched): kernel chosen, grid within one round of two blocks per CU, LDS within the CU's 160 KB
    {
        struct Shape { const char *what; int in, n, out[3], g, pair, norm; };
        const Shape shapes[] = {
            {"7B q|k|v", 4096, 3, {4096, 4096, 4096}, 128, 0, 1},   {"7B wo", 4096, 1, {4096, 0, 0}, 128, 0, 0},
            {"7B w1|w3", 4096, 2, {11008, 11008, 0}, 128, 1, 1},    {"7B w2", 11008, 1, {4096, 0, 0}, 128, 0, 0},
            {"13B q|k|v", 5120, 3, {5120, 5120, 5120}, 128, 0, 1},  {"13B wo", 5120, 1, {5120, 0, 0}, 128, 0, 0},
            {"13B w1|w3", 5120, 2, {13824, 13824, 0}, 128, 1, 1},   {"13B w2", 13824, 1, {5120, 0, 0}, 128, 0, 0},
            {"70B q|k|v", 8192, 3, {8192, 1024, 1024}, 64, 0, 1},   {"70B wo", 8192, 1, {8192, 0, 0}, 64, 0, 0},
            {"70B w1|w3", 8192, 2, {28672, 28672, 0}, 64, 1, 1},    {"70B w2", 28672, 1, {8192, 0, 0}, 64, 0, 0},
            {"ragged", 4160, 1, {72, 0, 0}, 32, 0, 0},              {"tiny", 256, 2, {64, 8, 0}, 32, 0, 1},
        };
        for (const Shape &sh : shapes) {
            char name[160];
            int32_t geo[4] = {0, 0, 0, 0};
            if (l2_q4_plan(sh.in, sh.out, sh.n, sh.g, sh.pair, sh.norm, name, sizeof name, geo) != L2_OK) {
                fprintf(stderr, "%s: %s\n", sh.what, l2_last_error());
                return 1;
            }
            REQUIRE(strlen(name) > 8);
            REQUIRE(geo[0] >= 1 && geo[0] <= 4 * 256 && geo[1] >= 64 && geo[1] <= 1024 && geo[2] >= 1);
            REQUIRE(geo[3] >= 0 && geo[3] <= 152 * 1024);
        }
        char name[8];
        int32_t geo[4];
        const int32_t bad_out[3] = {12, 0, 0};
        REQUIRE(l2_q4_plan(4096, bad_out, 1, 128, 0, 0, name, sizeof name, geo) != L2_OK);   // out not a multiple of 8
        REQUIRE(l2_q4_plan(4100, shapes[1].out, 1, 128, 0, 0, name, sizeof name, geo) != L2_OK);
        REQUIRE(l2_q4_plan(4096, shapes[1].out, 4, 128, 0, 0, name, sizeof name, geo) != L2_OK);
    }

    // tokenizer (src/tokenizer.rs:22-108): every token, round trips, buffers that are too small
    l2_tokenizer *tk = nullptr;
    REQUIRE(l2_tokenizer_open("/nonexistent/tokenizer.bin", 32000, &tk) != L2_OK);
    REQUIRE(l2_tokenizer_open(argv[1], 32000, &tk) == L2_OK);
    REQUIRE(l2_tokenizer_vocab_size(tk) == 32000);
    size_t total = 0;
    for (int id = 0; id < 32000; id++) {
        const char *str = nullptr;
        int len = 0;
        float score = 0.f;
        REQUIRE(l2_tokenizer_token(tk, id, &str, &len, &score) == L2_OK && str && len >= 0);
        total += (size_t)len;
    }
    REQUIRE(total > 32000);
    const char *str = nullptr;
    int len = 0;
    REQUIRE(l2_tokenizer_token(tk, 32000, &str, &len, &f) != L2_OK);
    REQUIRE(l2_tokenizer_token(tk, -1, &str, &len, &f) != L2_OK);
    const char *texts[] = {"", " ", "Hello, world", "The quick brown fox jumps over the lazy dog.",
                           "na\xC3\xAFve caf\xC3\xA9 \xE2\x82\xAC 10", "\xF0\x9F\x98\x80 emoji", "\xFF\xFE not utf-8",
                           "aaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaa"};
    for (const char *text : texts) {
        std::vector<int32_t> ids(strlen(text) + 8);
        int n = -1;
        rc = l2_tokenizer_encode(tk, text, ids.data(), (int)ids.size(), &n);
        if (rc == L2_OK) {
            REQUIRE(n >= 0 && n <= (int)ids.size());
            std::string back;
            for (int i = 0; i < n; i++) {
                REQUIRE(l2_tokenizer_token(tk, ids[(size_t)i], &str, &len, &f) == L2_OK);
                back.append(str, (size_t)len);
            }
            REQUIRE(back == text);
            if (n > 1) {
                int n2 = 0;
                REQUIRE(l2_tokenizer_encode(tk, text, ids.data(), n - 1, &n2) != L2_OK); // capacity too small
            }
        }
    }
    l2_tokenizer_free(tk);

    // Random and sample (src/util.rs:55-123)
    l2_random *r = nullptr;
    REQUIRE(l2_random_new(7, 0, &r) == L2_OK);
    std::vector<float> p(1000);
    double sum = 0;
    for (size_t i = 0; i < p.size(); i++) sum += (p[i] = 1.0f + (float)(i % 7));
    for (float &v : p) v = (float)(v / sum);
    for (int i = 0; i < 10000; i++) {
        const float u = l2_random_f32(r);
        REQUIRE(u >= 0.f && u < 1.f);
        const int k = l2_random_sample(r, p.data(), (int)p.size());
        REQUIRE(k >= 0 && k < (int)p.size());
    }
    REQUIRE(l2_random_sample(r, p.data(), 1) == 0);
    l2_random_free(r);
    REQUIRE(l2_random_new(0, 1, &r) == L2_OK); // seeded from the clock
    (void)l2_random_f32(r);
    l2_random_free(r);

    REQUIRE(l2_kernel_class_count() > 0);
    for (int c = 0; c < l2_kernel_class_count(); c++) REQUIRE(l2_kernel_class_name(c) != nullptr);
    puts("ok");
    return 0;
}
