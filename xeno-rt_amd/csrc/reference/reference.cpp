// Plain C++ references of the kernel library's operations: the same arguments as the xrt_* entry points,
// float32 in host memory, one loop nest per formula, no HIP. They are what each kernel is held against in
// the tests (beside the Python stand-in), and they build for the CPU alone, also under the host sanitizers.
//
// Formulas of the reference implementation (crates/ of XENO-CORPORATION/xeno-rt):
//   rmsnorm      xrt-kernels/src/cpu/rmsnorm.rs:26-43     y = (x * 1/sqrt(mean(x^2) + eps)) * w
//   rotation     xrt-kernels/src/cpu/rope.rs:10-16, 59-89 theta_i = base^(2i/d); angle = pos * scale / theta_i;
//                                                          (x0, x1) -> (x0 cos - x1 sin, x0 sin + x1 cos), pairs (i, i + d/2)
//   silu         xrt-kernels/src/cpu/silu.rs:1-3, 22-24   z / (1 + exp(-z)); swiglu = silu(gate) * up
//   softmax      xrt-kernels/src/cpu/softmax.rs:14-109    exp(x - max) / sum
//   matvec       xrt-kernels/src/cpu/matmul.rs:153-167    out[r] = sum_c w[r][c] x[c]
//   head norm    xrt-models/src/llama.rs:1025-1040        rmsnorm of every head with one weight [head_dim]
//   attention    xrt-models/src/llama.rs:504-574          scores over keys 0..pos of head h / group, softmax, weighted values
//   sampling     xrt-runtime/src/sampler.rs:56-200        penalty, greedy, temperature, top-k, top-p, inverse CDF
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <vector>

#include "reference.h"

namespace {

constexpr int BLOCK = 64;           // tokens of a cache block

// Where the elements of a cache block lie. Head sizes that are no multiple of 32: keys [token][dim], values
// [dim][token]. Multiples of 32: in the order in which a wavefront of the decode kernel holds the block, found here by
// walking that order: tiles of 64 lanes' pieces of 8 elements, lane (r, c) at place r + 16 c.
//   keys:   for each half g of the block, each score tile t of it, each 32 dims s: lane (r, c) has dims
//           32 s + 8 c .. + 7 of key 32 g + 8 (r / 4) + 4 t + r % 4;
//   values: for each half g, each 16 dims u: lane (r, c) has tokens 32 g + 8 c .. + 7 of dim 16 u + r.
struct BlockOrder {
    std::vector<int> key, value;     // [token * head_dim + dim], [dim * BLOCK + token] -> element offset in the block
    explicit BlockOrder(int head_dim) : key((size_t)BLOCK * head_dim), value((size_t)BLOCK * head_dim) {
        if (head_dim % 32 != 0) {
            std::iota(key.begin(), key.end(), 0);
            std::iota(value.begin(), value.end(), 0);
            return;
        }
        int at = 0;
        for (int g = 0; g < 2; ++g)
            for (int t = 0; t < 2; ++t)
                for (int s = 0; s < head_dim / 32; ++s)
                    for (int c = 0; c < 4; ++c)
                        for (int r = 0; r < 16; ++r)
                            for (int e = 0; e < 8; ++e)
                                key[(size_t)(32 * g + 8 * (r / 4) + 4 * t + r % 4) * head_dim + 32 * s + 8 * c + e] = at++;
        at = 0;
        for (int g = 0; g < 2; ++g)
            for (int u = 0; u < head_dim / 16; ++u)
                for (int c = 0; c < 4; ++c)
                    for (int r = 0; r < 16; ++r)
                        for (int e = 0; e < 8; ++e)
                            value[(size_t)(16 * u + r) * BLOCK + 32 * g + 8 * c + e] = at++;
    }
};

float activation(float z, int code) {
    (void)code;                      // XRT_ACT_SILU is the only one
    return z / (1.0f + std::exp(-z));
}

}  // namespace

extern "C" {

int xrt_ref_block_tokens(void) { return BLOCK; }

int xrt_ref_cache_key_offset(int token, int dim, int head_dim) { return BlockOrder(head_dim).key[(size_t)token * head_dim + dim]; }
int xrt_ref_cache_value_offset(int dim, int token, int head_dim) { return BlockOrder(head_dim).value[(size_t)dim * BLOCK + token]; }

void xrt_ref_embed(const float* table, const int* ids, float* out, int tokens, int hidden) {
    for (int t = 0; t < tokens; ++t)
        for (int i = 0; i < hidden; ++i) out[(long)t * hidden + i] = table[(long)ids[t] * hidden + i];
}

void xrt_ref_add(float* residual, const float* delta, long count) {
    for (long i = 0; i < count; ++i) residual[i] += delta[i];
}

void xrt_ref_rmsnorm(const float* x, const float* weight, float eps, float* out, const int* rows, int n_rows, int hidden) {
    for (int r = 0; r < n_rows; ++r) {
        const float* row = x + (long)(rows ? rows[r] : r) * hidden;
        float sum = 0.f;
        for (int i = 0; i < hidden; ++i) sum += row[i] * row[i];
        const float inv_rms = 1.0f / std::sqrt(sum / (float)hidden + eps);
        for (int i = 0; i < hidden; ++i) out[(long)r * hidden + i] = (row[i] * inv_rms) * weight[i];
    }
}

// mode 0 store, 1 accumulate, 2 (| activation << 8) gated with w = [gate rows | up rows]
void xrt_ref_linear(const float* a, const float* w, float* out, int M, int N, int K, int mode) {
    const int kind = mode & 255, code = mode >> 8;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float sum = 0.f, up = 0.f;
            for (int k = 0; k < K; ++k) sum += a[(long)m * K + k] * w[(long)n * K + k];
            if (kind == 2)
                for (int k = 0; k < K; ++k) up += a[(long)m * K + k] * w[((long)N + n) * K + k];
            float& dst = out[(long)m * N + n];
            if (kind == 0) dst = sum;
            else if (kind == 1) dst += sum;
            else dst = activation(sum, code) * up;
        }
}

void xrt_ref_qkv_prepare(float* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const int* positions,
                         const int* slots, const float* q_norm, const float* k_norm, float norm_eps,
                         const float* rope_theta, int rope_dim, float rope_scale, float* k_cache, float* v_cache,
                         const int* block_table, int table_stride, int n_blocks) {
    const int width = (n_heads + 2 * n_kv_heads) * head_dim;
    for (int t = 0; t < tokens; ++t) {
        float* row = qkv + (long)t * width;
        for (int head = 0; head < n_heads + n_kv_heads; ++head) {          // queries, then keys; values are left as they are
            float* h = row + (long)head * head_dim;
            const float* gain = head < n_heads ? q_norm : k_norm;
            if (gain) {
                float sum = 0.f;
                for (int d = 0; d < head_dim; ++d) sum += h[d] * h[d];
                const float inv_rms = 1.0f / std::sqrt(sum / (float)head_dim + norm_eps);
                for (int d = 0; d < head_dim; ++d) h[d] = h[d] * inv_rms * gain[d];
            }
            if (rope_theta) {
                const int half = std::min(rope_dim, head_dim) / 2;
                for (int i = 0; i < half; ++i) {
                    const float angle = (float)positions[t] * rope_scale / rope_theta[i];
                    const float s = std::sin(angle), c = std::cos(angle);
                    const float x0 = h[i], x1 = h[half + i];
                    h[i] = x0 * c - x1 * s;
                    h[half + i] = x0 * s + x1 * c;
                }
            }
        }
        if (!k_cache || slots[t] < 0) continue;
        const BlockOrder order(head_dim);
        const int block = block_table[(long)slots[t] * table_stride + positions[t] / BLOCK];
        if (block < 0 || block >= n_blocks) continue;
        const int within = positions[t] % BLOCK;
        for (int kv = 0; kv < n_kv_heads; ++kv)
            for (int d = 0; d < head_dim; ++d) {
                const long base = ((long)block * n_kv_heads + kv) * BLOCK * head_dim;
                k_cache[base + order.key[(size_t)within * head_dim + d]] = row[(long)(n_heads + kv) * head_dim + d];
                v_cache[base + order.value[(size_t)d * BLOCK + within]] = row[(long)(n_heads + n_kv_heads + kv) * head_dim + d];
            }
    }
}

void xrt_ref_attention(const float* qkv, int tokens, int n_heads, int n_kv_heads, int head_dim, const float* k_cache,
                       const float* v_cache, const int* block_table, int table_stride, const int* positions,
                       const int* slots, float* out, float scale, int window, const float* distance_slopes) {
    const int width = (n_heads + 2 * n_kv_heads) * head_dim, group = n_heads / n_kv_heads;
    const BlockOrder order(head_dim);
    for (int t = 0; t < tokens; ++t)
        for (int head = 0; head < n_heads; ++head) {
            float* dst = out + ((long)t * n_heads + head) * head_dim;
            std::fill(dst, dst + head_dim, 0.f);
            if (slots[t] < 0) continue;
            const int kv = head / group, pos = positions[t];
            const int first = window > 0 ? std::max(0, pos - window + 1) : 0;
            const float* q = qkv + (long)t * width + (long)head * head_dim;
            std::vector<float> scores(pos + 1 - first);
            for (int key = first; key <= pos; ++key) {
                const int block = block_table[(long)slots[t] * table_stride + key / BLOCK];
                const float* k = k_cache + ((long)block * n_kv_heads + kv) * BLOCK * head_dim;
                const int* place = &order.key[(size_t)(key % BLOCK) * head_dim];
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot += q[d] * k[place[d]];
                scores[key - first] = dot * scale + (distance_slopes ? distance_slopes[head] * (float)(key - pos) : 0.f);
            }
            const float largest = *std::max_element(scores.begin(), scores.end());
            float total = 0.f;
            for (float& s : scores) { s = std::exp(s - largest); total += s; }
            for (int key = first; key <= pos; ++key) {
                const int block = block_table[(long)slots[t] * table_stride + key / BLOCK];
                const float* v = v_cache + ((long)block * n_kv_heads + kv) * head_dim * BLOCK;
                const float p = scores[key - first] / total;
                for (int d = 0; d < head_dim; ++d) dst[d] += p * v[order.value[(size_t)d * BLOCK + key % BLOCK]];
            }
        }
}

// sampler.rs: penalty on the tokens seen (logit > 0 ? / pen : * pen, only if pen > 1); temperature <= 1e-5: the first
// index of the maximum; else keep the k largest (0: all; ties at the k-th are all kept, as the kernels do),
// weights exp((logit - max) / T), keep the heaviest whose mass reaches top_p of the whole, draw by the
// inverse CDF over token ids with the row's uniform number.
void xrt_ref_sample(const float* logits, int rows, int vocab, int* out, const float* temperature, const int* top_k,
                    const float* top_p, const float* penalty, int* history, const int* history_spans,
                    const int* append_at, const float* uniforms) {
    for (int r = 0; r < rows; ++r) {
        std::vector<float> row(logits + (long)r * vocab, logits + (long)(r + 1) * vocab);
        if (penalty[r] > 1.0f) {
            std::vector<char> seen(vocab, 0);
            for (int i = history_spans[2 * r]; i < history_spans[2 * r + 1]; ++i)
                if (history[i] >= 0 && history[i] < vocab) seen[history[i]] = 1;
            for (int i = 0; i < vocab; ++i)
                if (seen[i]) row[i] = row[i] > 0.f ? row[i] / penalty[r] : row[i] * penalty[r];
        }
        int best = 0;
        float best_value = -INFINITY;
        bool any = false;
        for (int i = 0; i < vocab; ++i)
            if (row[i] > best_value) { best = i; best_value = row[i]; any = true; }
        if (!any) best = 0;
        int pick = best;
        if (temperature[r] > 1e-5f) {
            const int k = top_k[r] > 0 && top_k[r] < vocab ? top_k[r] : vocab;
            std::vector<float> sorted(row);
            std::nth_element(sorted.begin(), sorted.begin() + (k - 1), sorted.end(), std::greater<float>());
            const float kth = sorted[k - 1];
            std::vector<double> weight(vocab);
            for (int i = 0; i < vocab; ++i) weight[i] = row[i] >= kth ? std::exp((double)(row[i] - best_value) / temperature[r]) : 0.0;
            if (top_p[r] < 1.0f) {
                std::vector<int> order(vocab);
                std::iota(order.begin(), order.end(), 0);
                std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return weight[a] > weight[b]; });
                const double whole = std::accumulate(weight.begin(), weight.end(), 0.0);
                double mass = 0.0, threshold = 0.0;
                for (int i : order) { mass += weight[i]; threshold = weight[i]; if (mass >= top_p[r] * whole) break; }
                for (double& x : weight) if (x < threshold) x = 0.0;
            }
            const double whole = std::accumulate(weight.begin(), weight.end(), 0.0);
            const double target = (double)uniforms[r] * whole;
            double running = 0.0;
            int last = -1;
            pick = -1;
            for (int i = 0; i < vocab && pick < 0; ++i)
                if (weight[i] > 0.0) { last = i; running += weight[i]; if (running > target) pick = i; }
            if (pick < 0) pick = last >= 0 ? last : best;
        }
        out[r] = pick;
        if (append_at && append_at[r] >= 0) history[append_at[r]] = pick;
    }
}

// element i of the random-weights stream `key` (weights/random_init.py of the package)
void xrt_ref_random_normal(float* out, long count, unsigned long long key, float scale, float offset) {
    auto mix = [](uint64_t v) {
        v += 0x9E3779B97F4A7C15ull;
        v = (v ^ (v >> 30)) * 0xBF58476D1CE4E5B9ull;
        v = (v ^ (v >> 27)) * 0x94D049BB133111EBull;
        return v ^ (v >> 31);
    };
    for (long i = 0; i < count; ++i) {
        const uint64_t base = key + (uint64_t)(2 * i) * 0x9E3779B97F4A7C15ull;
        int sum = 0;
        for (uint64_t word : {mix(base), mix(base + 0x9E3779B97F4A7C15ull)})
            for (int f = 0; f < 6; ++f) sum += (int)((word >> (10 * f)) & 1023u);
        volatile float product = (float)(2 * sum - 12 * 1023) * scale;      // rounded before the addition, as everywhere
        out[i] = offset != 0.f ? product + offset : product;
    }
}

// w [rows][K] into tiles of 16 rows x 32 columns (csrc/packing.h); kind 1 tiles, 2 gate/up pairs, 3 rotary pairs
void xrt_ref_pack_weight(const float* w, float* packed, int rows, int K, int kind, int gated_n, int head_dim, int rotated_heads) {
    const long padded = ((long)rows + 15) / 16 * 16;
    for (long p = 0; p < padded; ++p) {
        long logical = p;
        if (kind == 2) {
            const long group = p / 16, within = p % 16;
            logical = within < 8 ? group * 8 + within : (long)gated_n + group * 8 + (within - 8);
        } else if (kind == 3 && p / head_dim < rotated_heads) {
            const long head = p / head_dim, within = p % head_dim;
            logical = head * head_dim + (within % 16 / 8) * (head_dim / 2) + within / 16 * 8 + within % 8;
        }
        for (int k = 0; k < K; ++k) {
            const long at = ((p / 16) * (K / 32) + k / 32) * 512 + ((k % 32 / 8) * 16 + p % 16) * 8 + k % 8;
            packed[at] = logical < rows ? w[logical * K + k] : 0.f;
        }
    }
}

}  // extern "C"
