// Host-side text surface of the token loop: the llama2.c-format tokenizer
// (src/tokenizer.rs:22-108, src/util.rs:29-37), the xorshift* generator and CDF
// sampler (src/util.rs:55-113), and generate() on strings
// (src/inference.rs:49-193, src/util.rs:116-128).  String work and the
// per-token sampling arithmetic run on the host, as they do in the reference;
// every transformer step goes through l2_forward / l2_generate_greedy.
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <chrono>
#include <string>
#include <unordered_map>
#include <vector>

#include "l2_internal.h"

struct l2_tokenizer {
    std::vector<std::string> vocab;
    std::vector<float> scores;
    int max_token_length = 0;
    // str_lookup (src/util.rs:29-37): first match among ids >= 260, else first match overall
    std::unordered_map<std::string, int> first_hi, first_any;
};

struct l2_random {
    uint64_t seed;
};

static int lookup(const l2_tokenizer *t, const std::string &s) {
    auto it = t->first_hi.find(s);
    if (it != t->first_hi.end()) return it->second;
    it = t->first_any.find(s);
    return it == t->first_any.end() ? -1 : it->second;
}

static bool valid_utf8(const std::string &s) {
    size_t i = 0;
    const size_t n = s.size();
    while (i < n) {
        const unsigned char c = (unsigned char)s[i];
        const size_t k = c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : (c >> 3) == 30 ? 4 : 0;
        if (k == 0 || i + k > n) return false;
        for (size_t j = 1; j < k; j++)
            if (((unsigned char)s[i + j] >> 6) != 2) return false;
        i += k;
    }
    return true;
}

extern "C" int l2_tokenizer_open(const char *path, int vocab_size, l2_tokenizer **out) {
    if (!path || !out || vocab_size <= 0) return l2_fail(L2_ERR_ARG, "l2_tokenizer_open: bad argument");
    FILE *f = fopen(path, "rb");
    if (!f) return l2_fail(L2_ERR_IO, "Failed to open %s", path);
    l2_tokenizer *t = new l2_tokenizer();
    int32_t mtl = 0;
    bool ok = fread(&mtl, 4, 1, f) == 1; // src/tokenizer.rs:29
    t->max_token_length = mtl;
    t->vocab.reserve(vocab_size);
    t->scores.reserve(vocab_size);
    for (int i = 0; ok && i < vocab_size; i++) { // :30-35
        float score;
        int32_t len;
        ok = fread(&score, 4, 1, f) == 1 && fread(&len, 4, 1, f) == 1 && len >= 0 && len < (1 << 20);
        if (!ok) break;
        std::string s((size_t)len, '\0');
        ok = len == 0 || fread(&s[0], 1, (size_t)len, f) == (size_t)len;
        if (ok && !valid_utf8(s)) ok = false; // read_str unwraps from_utf8 (src/util.rs:16-20)
        t->scores.push_back(score);
        t->vocab.push_back(std::move(s));
    }
    fclose(f);
    if (!ok) {
        delete t;
        return l2_fail(L2_ERR_FORMAT, "%s: not a tokenizer file with %d entries", path, vocab_size);
    }
    for (int i = 0; i < vocab_size; i++) {
        t->first_any.emplace(t->vocab[i], i);
        if (i >= 260) t->first_hi.emplace(t->vocab[i], i);
    }
    *out = t;
    return L2_OK;
}

extern "C" void l2_tokenizer_free(l2_tokenizer *t) { delete t; }

extern "C" int l2_tokenizer_vocab_size(const l2_tokenizer *t) { return t ? (int)t->vocab.size() : 0; }

extern "C" int l2_tokenizer_token(const l2_tokenizer *t, int id, const char **str, int *len, float *score) {
    if (!t || id < 0 || id >= (int)t->vocab.size()) return l2_fail(L2_ERR_RANGE, "token id %d", id);
    if (str) *str = t->vocab[id].data();
    if (len) *len = (int)t->vocab[id].size();
    if (score) *score = t->scores[id];
    return L2_OK;
}

// Tokenizer::bpe_encode (src/tokenizer.rs:46-108)
static int bpe_encode(const l2_tokenizer *t, const std::string &text, std::vector<int> &tokens) {
    tokens.clear();
    if (!valid_utf8(text)) return l2_fail(L2_ERR_ARG, "text is not UTF-8");
    // first every character on its own (:53-60)
    for (size_t i = 0; i < text.size();) {
        const unsigned char c = (unsigned char)text[i];
        const int n = c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : 4;
        const int id = lookup(t, text.substr(i, n));
        if (id < 0) return l2_fail(L2_ERR_ARG, "character at byte %zu is not in the vocabulary", i); // expect("not good")
        tokens.push_back(id);
        i += n;
    }
    if (tokens.empty()) return l2_fail(L2_ERR_ARG, "empty text"); // the reference's 0..len-1 underflows here
    std::string buf;
    for (;;) { // merge the best consecutive pair each round (:63-107)
        float best_score = -1e10f;
        int best_id = 0, best_idx = -1;
        for (size_t i = 0; i + 1 < tokens.size(); i++) {
            buf.assign(t->vocab[tokens[i]]);
            buf.append(t->vocab[tokens[i + 1]]);
            const int id = lookup(t, buf);
            if (id >= 0 && t->scores[id] > best_score) {
                best_score = t->scores[id];
                best_id = id;
                best_idx = (int)i;
            }
        }
        if (best_idx < 0) return L2_OK;
        tokens[best_idx] = best_id;
        tokens.erase(tokens.begin() + best_idx + 1);
    }
}

extern "C" int l2_tokenizer_encode(const l2_tokenizer *t, const char *text, int32_t *ids, int cap, int *n) {
    if (!t || !text || !n) return l2_fail(L2_ERR_ARG, "l2_tokenizer_encode: null argument");
    std::vector<int> tokens;
    L2_TRY(bpe_encode(t, text, tokens));
    *n = (int)tokens.size();
    if (!ids || cap < *n) return ids ? l2_fail(L2_ERR_ARG, "ids holds %d, %d needed", cap, *n) : L2_OK;
    for (int i = 0; i < *n; i++) ids[i] = tokens[i];
    return L2_OK;
}

// Random (src/util.rs:55-83)
extern "C" int l2_random_new(uint64_t seed, int from_clock, l2_random **out) {
    if (!out) return l2_fail(L2_ERR_ARG, "null argument");
    l2_random *r = new l2_random();
    r->seed = from_clock ? (uint64_t)std::chrono::duration_cast<std::chrono::seconds>(
                               std::chrono::system_clock::now().time_since_epoch())
                               .count()
                         : seed;
    *out = r;
    return L2_OK;
}

extern "C" void l2_random_free(l2_random *r) { delete r; }

static uint32_t random_u32(l2_random *r) { // :71-77
    r->seed ^= r->seed >> 12;
    r->seed ^= r->seed << 25;
    r->seed ^= r->seed >> 27;
    return (uint32_t)((r->seed * 0x2545F4914F6CDD1Dull) >> 32);
}

extern "C" float l2_random_f32(l2_random *r) { return r ? (float)(random_u32(r) >> 8) / 16777216.0f : 0.f; } // :79-82

// Random::sample (src/util.rs:102-113)
extern "C" int l2_random_sample(l2_random *r, const float *probabilities, int n) {
    if (!r || !probabilities || n < 1) return -1;
    const float x = l2_random_f32(r);
    float cdf = 0.0f;
    for (int i = 0; i < n; i++) {
        cdf += probabilities[i];
        if (x < cdf) return i;
    }
    return n - 1;
}

// softmax (src/models.rs:68-81) on the host, for temperature sampling only
static void softmax_host(float *x, int n) {
    float max_val = x[0];
    for (int i = 0; i < n; i++) max_val = fmaxf(max_val, x[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; i++) {
        x[i] = expf(x[i] - max_val);
        sum += x[i];
    }
    for (int i = 0; i < n; i++) x[i] /= sum;
}

// get_token (src/util.rs:116-123): after BOS, a leading space is stripped
static const char *token_text(const l2_tokenizer *t, int token, int next, int *len) {
    const std::string &s = t->vocab[next];
    if (token == 1 && !s.empty() && s[0] == ' ') {
        *len = (int)s.size() - 1;
        return s.data() + 1;
    }
    *len = (int)s.size();
    return s.data();
}

// char::is_whitespace (the White_Space property), which str::trim uses (src/inference.rs:63)
static bool is_unicode_space(uint32_t c) {
    return (c >= 0x09 && c <= 0x0D) || c == 0x20 || c == 0x85 || c == 0xA0 || c == 0x1680 ||
           (c >= 0x2000 && c <= 0x200A) || c == 0x2028 || c == 0x2029 || c == 0x202F || c == 0x205F || c == 0x3000;
}

// The code point that starts at byte i of valid UTF-8, and its length in bytes.
static uint32_t utf8_at(const std::string &s, size_t i, size_t *len) {
    const unsigned char c = (unsigned char)s[i];
    const size_t k = c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : 4;
    uint32_t cp = k == 1 ? c : (uint32_t)(c & (0xFFu >> (k + 1)));
    for (size_t j = 1; j < k; j++) cp = (cp << 6) | ((unsigned char)s[i + j] & 0x3Fu);
    *len = k;
    return cp;
}

static std::string trim_unicode(const std::string &p) {
    size_t a = 0, b = p.size(), k;
    while (a < b && is_unicode_space(utf8_at(p, a, &k))) a += k;
    while (b > a) {
        size_t q = b - 1; // start of the last character
        while (q > a && ((unsigned char)p[q] >> 6) == 2) q--;
        if (!is_unicode_space(utf8_at(p, q, &k))) break;
        b = q;
    }
    return p.substr(a, b - a);
}

extern "C" int l2_generate(l2_model *m, l2_state *s, const l2_tokenizer *t, const char *prompt, int steps,
                           l2_random *rng, float temperature, int print_tokens, char *out, size_t out_cap,
                           int *n_tokens, int64_t *ms) {
    if (!m || !s || !t || !prompt || !n_tokens || !ms || steps < 0) return l2_fail(L2_ERR_ARG, "l2_generate: bad argument");
    if (temperature != 0.0f && !rng) return l2_fail(L2_ERR_ARG, "l2_generate: sampling needs a Random");
    l2_dims d;
    L2_TRY(l2_model_dims(m, &d));
    if ((int)t->vocab.size() < d.vocab_size) return l2_fail(L2_ERR_ARG, "tokenizer has %zu entries, the model %d", t->vocab.size(), d.vocab_size);
    // prompt: " " + trim (src/inference.rs:62-67)
    std::vector<int> prompt_tokens;
    {
        const std::string p(prompt);
        if (!valid_utf8(p)) return l2_fail(L2_ERR_ARG, "prompt is not UTF-8");
        if (!p.empty()) L2_TRY(bpe_encode(t, " " + trim_unicode(p), prompt_tokens));
    }
    const int n_prompt = (int)prompt_tokens.size();
    const std::vector<int32_t> prompt32(prompt_tokens.begin(), prompt_tokens.end());
    std::vector<int32_t> ids((size_t)(steps > 0 ? steps : 1));
    const bool prefill = l2_prefill_supported(m) != 0;
    size_t used = 0;
    // one token string of get_token (src/util.rs:116-123): printed at once (print_token flushes, :125-128),
    // and, for the strings the reference returns, appended to `out`
    auto emit = [&](int token, int next, bool returned) -> int {
        int len;
        const char *str = token_text(t, token, next, &len);
        if (print_tokens) {
            fwrite(str, 1, (size_t)len, stdout);
            fflush(stdout);
        }
        if (!returned) return L2_OK;
        if (out) {
            if (used + (size_t)len + 1 > out_cap) return l2_fail(L2_ERR_ARG, "output buffer of %zu bytes is too small", out_cap);
            memcpy(out + used, str, (size_t)len);
            out[used + len] = '\0';
        }
        used += (size_t)len + 1;
        return L2_OK;
    };
    int n = 0;
    const auto t0 = std::chrono::system_clock::now(); // time_in_ms, :72
    if (temperature == 0.0f && !print_tokens) {
        // nothing is wanted before the end: the whole loop stays on the device
        double ms_loop = 0;
        L2_TRY(l2_generate_greedy(m, s, prompt32.data(), n_prompt, steps, prefill, ids.data(), &n, &ms_loop));
        const int first_pos = prefill ? l2_prefill_ladder_end(n_prompt) : 0; // the ladder may pass `steps`
        int token = first_pos == 0 ? 1 : prompt32[first_pos - 1];
        for (int i = 0; i < n; i++) {
            L2_TRY(emit(token, ids[i], true));
            token = ids[i];
        }
    } else {
        // the loop on the host, a token at a time, so that every string is printed when it exists and the
        // sampler sees the logits (:141-190)
        L2_TRY(l2_state_reset(s));
        int pos = 0;
        if (prefill) { // :16-44, :78-127
            std::vector<int32_t> toks(64), poss(64);
            for (int A = 64; A >= 2; A /= 2)
                while (pos + A < n_prompt) {
                    for (int i = 0; i < A; i++) {
                        toks[i] = pos == 0 ? 1 : prompt32[pos - 1];
                        poss[i] = pos++;
                        L2_TRY(emit(toks[i], toks[i], false)); // :37-40
                    }
                    L2_TRY(l2_forward(m, s, toks.data(), poss.data(), A, nullptr));
                }
        }
        int32_t token = pos == 0 ? 1 : prompt32[pos - 1];
        L2_TRY(emit(token, token, false)); // :134-137
        std::vector<float> logits(temperature != 0.0f ? (size_t)d.vocab_size : 0);
        while (pos < steps) {
            const int32_t p32 = pos;
            int32_t next = 0;
            if (temperature == 0.0f) {
                L2_TRY(l2_decode_greedy(m, s, token, p32, &next)); // :160-162, argmax on the device
                if (pos < n_prompt) next = prompt32[pos];
            } else {
                L2_TRY(l2_forward(m, s, &token, &p32, 1, logits.data()));
                if (pos < n_prompt) {
                    next = prompt32[pos];
                } else {
                    for (int q = 0; q < d.vocab_size; q++) logits[q] /= temperature; // :166-168
                    softmax_host(logits.data(), d.vocab_size);
                    next = l2_random_sample(rng, logits.data(), d.vocab_size);
                }
            }
            L2_TRY(emit(token, next, true)); // :178-182
            ids[n++] = next;
            token = next;
            pos++;
        }
    }
    const auto t1 = std::chrono::system_clock::now();
    *ms = std::chrono::duration_cast<std::chrono::milliseconds>(t1 - t0).count();
    *n_tokens = n;
    return L2_OK;
}
