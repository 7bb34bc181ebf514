// Runs every plain C++ reference on small inputs whose results are known, so that a build under the host
// sanitizers (-fsanitize=address,undefined) walks all of their loops. Exit status 0: every check held.
#include <cmath>
#include <cstdio>
#include <vector>

#include "reference.h"

static int failures = 0;
static void check(bool ok, const char* what) {
    if (!ok) { std::printf("FAILED: %s\n", what); ++failures; }
}
static bool close_to(float a, float b, float tolerance = 1e-5f) { return std::fabs(a - b) <= tolerance * (1.0f + std::fabs(b)); }

int main() {
    {   // rmsnorm: the vector of the reference's own test (tests/kernels_test.rs:75-91)
        const float x[4] = {1, 2, 3, 4}, w[4] = {1, 1.5f, 2, 2.5f};
        float y[4];
        xrt_ref_rmsnorm(x, w, 1e-5f, y, nullptr, 1, 4);
        const float inv = 1.0f / std::sqrt(7.5f + 1e-5f);
        check(close_to(y[0], inv) && close_to(y[1], 3 * inv) && close_to(y[2], 6 * inv) && close_to(y[3], 10 * inv), "rmsnorm");
        const int rows[2] = {0, 0};
        float twice[8];
        xrt_ref_rmsnorm(x, w, 1e-5f, twice, rows, 2, 4);
        check(twice[5] == y[1], "rmsnorm of picked rows");
    }
    {   // products: store, accumulate, gated
        const float a[2 * 3] = {1, 2, 3, -1, 0, 1}, w[4 * 3] = {1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1};
        float out[2 * 4] = {};
        xrt_ref_linear(a, w, out, 2, 4, 3, 0);
        check(out[0] == 1 && out[1] == 2 && out[2] == 3 && out[3] == 6 && out[4] == -1 && out[7] == 0, "linear store");
        xrt_ref_linear(a, w, out, 2, 4, 3, 1);
        check(out[3] == 12 && out[4] == -2, "linear accumulate");
        float gated[2 * 2];
        xrt_ref_linear(a, w, gated, 2, 2, 3, 2);
        check(close_to(gated[0], 1.0f / (1.0f + std::exp(-1.0f)) * 3.0f) && close_to(gated[1], 2.0f / (1.0f + std::exp(-2.0f)) * 6.0f), "linear gated");
    }
    {   // embedding and add
        const float table[3 * 2] = {0, 1, 10, 11, 20, 21};
        const int ids[2] = {2, 0};
        float out[4];
        xrt_ref_embed(table, ids, out, 2, 2);
        check(out[0] == 20 && out[1] == 21 && out[2] == 0 && out[3] == 1, "embed");
        const float delta[4] = {1, 1, 1, 1};
        xrt_ref_add(out, delta, 4);
        check(out[0] == 21 && out[3] == 2, "add");
    }
    {   // q/k/v preparation and attention: 2 query heads on 1 key/value head of 4 dims, two tokens of one sequence
        const int nh = 2, nkv = 1, hd = 4, tokens = 2, width = (nh + 2 * nkv) * hd;
        std::vector<float> qkv(tokens * width);
        for (size_t i = 0; i < qkv.size(); ++i) qkv[i] = 0.1f * (float)((i * 7) % 11) - 0.4f;
        const std::vector<float> before(qkv);
        const int positions[2] = {0, 1}, slots[2] = {0, 0}, table[1] = {0};
        const float theta[2] = {1.0f, 100.0f};
        std::vector<float> k_cache(64 * hd, 0.f), v_cache(64 * hd, 0.f);
        xrt_ref_qkv_prepare(qkv.data(), tokens, nh, nkv, hd, positions, slots, nullptr, nullptr, 0.f, theta, hd, 1.0f,
                            k_cache.data(), v_cache.data(), table, 1, 1);
        bool identity = true;                                   // position 0: no rotation
        for (int i = 0; i < width; ++i) identity = identity && qkv[i] == before[i];
        check(identity, "rotation at position 0");
        const float* q1 = &before[width], *r1 = &qkv[width];    // position 1, first pair of the first head: angle 1
        check(close_to(r1[0], q1[0] * std::cos(1.0f) - q1[2] * std::sin(1.0f)) && close_to(r1[2], q1[0] * std::sin(1.0f) + q1[2] * std::cos(1.0f)), "rotation pairs (i, i + d/2)");
        check(k_cache[1 * hd + 0] == qkv[width + nh * hd] && v_cache[0 * 64 + 1] == before[width + (nh + nkv) * hd], "cache holds rotated keys and raw values");
        // heads of a multiple of 32: the order of the decode kernel's operands. Worked out by hand: key 13 is row 5 of
        // score tile 1 of the first half, dims 16 .. 23 are lane group 2 of the first 32: tile (0 * 2 + 1) * 2 + 0,
        // place 5 + 32; dim 21 of the value of token 45: tile 1 * 4 + 1, row 5, tokens 40 .. 47 are lane group 1
        check(xrt_ref_cache_key_offset(13, 21, 64) == (2 * 64 + 37) * 8 + 5 && xrt_ref_cache_value_offset(21, 45, 64) == (5 * 64 + 5 + 16) * 8 + 5 &&
              xrt_ref_cache_key_offset(13, 21, 48) == 13 * 48 + 21 && xrt_ref_cache_value_offset(21, 45, 48) == 21 * 64 + 45, "order of a cache block");
        std::vector<float> out(tokens * nh * hd);
        xrt_ref_attention(qkv.data(), tokens, nh, nkv, hd, k_cache.data(), v_cache.data(), table, 1, positions, slots, out.data(), 0.5f, 0, nullptr);
        bool first_is_value = true;                             // one key: the output is its value
        for (int d = 0; d < hd; ++d) first_is_value = first_is_value && close_to(out[d], before[(nh + nkv) * hd + d]);
        check(first_is_value, "attention over one key");
        xrt_ref_attention(qkv.data(), tokens, nh, nkv, hd, k_cache.data(), v_cache.data(), table, 1, positions, slots, out.data(), 0.5f, 1, nullptr);
        bool windowed = true;                                   // a window of one: every token sees itself alone
        for (int d = 0; d < hd; ++d) windowed = windowed && close_to(out[nh * hd + d], before[width + (nh + nkv) * hd + d]);
        check(windowed, "attention window");
        const std::vector<float> steep(nh, 200.0f);              // scores fall by 200 per position of distance: again itself alone
        xrt_ref_attention(qkv.data(), tokens, nh, nkv, hd, k_cache.data(), v_cache.data(), table, 1, positions, slots, out.data(), 0.5f, 0, steep.data());
        bool biased = true;
        for (int d = 0; d < hd; ++d) biased = biased && close_to(out[nh * hd + d], before[width + (nh + nkv) * hd + d]);
        check(biased, "attention scores biased by distance");
        const float gain[4] = {1, 1, 1, 1};
        xrt_ref_qkv_prepare(qkv.data(), tokens, nh, nkv, hd, positions, slots, gain, gain, 0.f, nullptr, 0, 1.0f, nullptr, nullptr, table, 1, 1);
        float squares = 0.f;
        for (int d = 0; d < hd; ++d) squares += qkv[d] * qkv[d];
        check(close_to(squares / hd, 1.0f, 1e-4f), "head norm");
    }
    {   // sampling: the reference's cases (tests/sampler_test.rs:101-127)
        const float logits[4] = {-1.0f, 0.5f, 3.25f, 2.0f};
        int out[1], history[1] = {1};
        const int spans[2] = {0, 1};
        float t = 0.f, p = 0.1f, pen = 1.0f, u = 0.5f;
        int k = 1;
        xrt_ref_sample(logits, 1, 4, out, &t, &k, &p, &pen, history, spans, nullptr, &u);
        check(out[0] == 2, "greedy");
        const float two[2] = {1.2f, 1.5f};
        pen = 2.0f;
        xrt_ref_sample(two, 1, 2, out, &t, &k, &p, &pen, history, spans, nullptr, &u);
        check(out[0] == 0, "penalty");
        t = 1.0f; k = 0; p = 1.0f; pen = 1.0f; u = 0.999f;
        xrt_ref_sample(logits, 1, 4, out, &t, &k, &p, &pen, history, spans, nullptr, &u);
        check(out[0] == 3, "the last token of the inverse CDF");
        k = 2; u = 0.999f;
        const int append[1] = {0};
        xrt_ref_sample(logits, 1, 4, out, &t, &k, &p, &pen, history, spans, append, &u);
        check(out[0] == 3 && history[0] == 3, "top-k keeps the two largest; the token is appended");
    }
    {   // random weights and packing
        float values[1000];
        xrt_ref_random_normal(values, 1000, 12345ull, 0.01f, 0.f);
        double mean = 0;
        for (float v : values) mean += v;
        check(std::fabs(mean / 1000) < 2.0, "random normal");
        const int rows = 20, K = 64;
        std::vector<float> w(rows * K), packed(32 * K, -1.f);
        for (size_t i = 0; i < w.size(); ++i) w[i] = (float)i;
        xrt_ref_pack_weight(w.data(), packed.data(), rows, K, 1, 0, 0, 0);
        check(packed[0] == 0 && packed[8] == (float)K && packed[(0 * 2 + 1) * 512 + 0] == 32.f && packed[(1 * 2 + 0) * 512 + 4 * 8] == 0.f, "packing in tiles");
        std::vector<float> pairs(32 * K);
        xrt_ref_pack_weight(w.data(), pairs.data(), 16, K, 2, 8, 0, 0);       // the first 16 rows as 8 gate rows and 8 up rows
        check(pairs[8 * 8] == w[8 * K], "packing gate with up rows");
    }
    if (failures == 0) std::printf("reference selftest ok\n");
    return failures == 0 ? 0 : 1;
}
