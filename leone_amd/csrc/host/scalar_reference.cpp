// A scalar single-precision reference of every kernel entry point, on host memory: one plain loop per
// operation, every sum taken left to right in float (attention's and the sampler's as the kernels' own rules
// say), the cache in the same paged layout as on the device.  It exists to be compared with: the kernels
// against it at rounding level, it against the double-precision formulas, a paged cache against a contiguous
// one bit for bit.  Nothing on the product path calls it (the reference keeps such a scalar backend beside its
// kernels: README.md:30, docs/oracle.md:16-21, crates/leone/src/cpu.rs:2928-3109).
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

#include "leone_host.h"

namespace {

// The cache layout of the device (keys [element / 8][token][8], values [token / 8][element][8] inside a
// page of one kv head).
inline long key_offset(int token, int element, int page_tokens) {
    return (static_cast<long>(element >> 3) * page_tokens + token) * 8 + (element & 7);
}
inline long value_offset(int token, int element, int head_dim) {
    return (static_cast<long>(token >> 3) * head_dim + element) * 8 + (token & 7);
}

}  // namespace

extern "C" {

// out[r] = table[tokens[r]]; an id outside the table gives a row of NaN.
int leone_ref_embed(const float* table, const int* tokens, float* out, int rows, int hidden, int vocab) {
    if (!table || !tokens || !out || rows <= 0 || hidden <= 0 || vocab <= 0) return LEONE_HOST_INVALID;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < hidden; ++c)
            out[static_cast<long>(r) * hidden + c] =
                (tokens[r] < 0 || tokens[r] >= vocab) ? std::numeric_limits<float>::quiet_NaN()
                                                      : table[static_cast<long>(tokens[r]) * hidden + c];
    return 0;
}

// x += delta (planes added in order) and y = (x * gain) / sqrt(mean(x^2) + eps); with `rows`, output row r is
// made from row rows[r] and x stays as it is (crates/leone/src/cpu.rs:1642-1663).
int leone_ref_add_rmsnorm(float* x, const float* delta, int planes, long plane, const float* gain, float eps,
                          float* y, const int* rows, int n_rows, int hidden) {
    if (!x || !gain || !y || n_rows <= 0 || hidden <= 0 || !(eps > 0.f)) return LEONE_HOST_INVALID;
    std::vector<float> v(hidden);
    for (int r = 0; r < n_rows; ++r) {
        const long in_row = rows ? rows[r] : r;
        float ss = 0.f;
        for (int c = 0; c < hidden; ++c) {
            float value = x[in_row * hidden + c];
            if (delta)
                for (int p = 0; p < planes; ++p) value += delta[p * plane + in_row * hidden + c];
            if (delta && !rows) x[in_row * hidden + c] = value;
            v[c] = value;
            ss = ss + value * value;
        }
        const float inv = 1.0f / std::sqrt(ss / static_cast<float>(hidden) + eps);
        for (int c = 0; c < hidden; ++c) y[static_cast<long>(r) * hidden + c] = (v[c] * gain[c]) * inv;
    }
    return 0;
}

// cos and sin of position * theta^(-2 i / rotary_dim), evaluated in double (crates/leone/src/cpu.rs:1721-1779).
int leone_ref_rope_table(float* cos_out, float* sin_out, double theta, int rotary_dim, int positions) {
    if (!cos_out || !sin_out || rotary_dim <= 0 || rotary_dim % 2 || positions <= 0 || !(theta > 0.0)) return LEONE_HOST_INVALID;
    const int pairs = rotary_dim / 2;
    for (int p = 0; p < positions; ++p)
        for (int i = 0; i < pairs; ++i) {
            const double angle = static_cast<double>(p) * std::pow(theta, -2.0 * i / rotary_dim);
            cos_out[static_cast<long>(p) * pairs + i] = static_cast<float>(std::cos(angle));
            sin_out[static_cast<long>(p) * pairs + i] = static_cast<float>(std::sin(angle));
        }
    return 0;
}

// Per-head RMSNorm of q and k (gains may be null), rotation of the head's first rotary_dim elements in half-split
// (pairing 0) or adjacent (pairing 1) pairs (tables [positions, rotary_dim / 2], may be null), q to q_out, k and
// v into the paged cache (crates/leone/src/backend.rs:2182-2208, crates/leone/src/cpu.rs:1765-1774).  The input
// may come in planes to be added up.
int leone_ref_qk_norm_rope_write(const float* qkv, int planes, long plane, float* q_out, float* k_pool, float* v_pool,
                                 const float* q_gain, const float* k_gain, float eps, const float* cos_table,
                                 const float* sin_table, int table_positions, int rotary_dim, int pairing,
                                 const int* positions,
                                 const int* row_entry, const int* block_table, int max_blocks, int rows, int q_heads,
                                 int kv_heads, int head_dim, int page_tokens, int write_cache) {
    if (!qkv || !q_out || !positions || rows <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 2)
        return LEONE_HOST_INVALID;
    if (write_cache && (!k_pool || !v_pool || !row_entry || !block_table || max_blocks <= 0 || page_tokens <= 0 ||
                        head_dim % 8 || page_tokens % 8))
        return LEONE_HOST_INVALID;
    if ((q_gain == nullptr) != (k_gain == nullptr) || (cos_table == nullptr) != (sin_table == nullptr)) return LEONE_HOST_INVALID;
    if (cos_table && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > head_dim || pairing < 0 || pairing > 1))
        return LEONE_HOST_INVALID;
    const int half = cos_table ? rotary_dim / 2 : 0;
    const long width = static_cast<long>(q_heads + 2 * kv_heads) * head_dim;
    std::vector<float> head(head_dim);
    for (int r = 0; r < rows; ++r) {
        const int pos = positions[r];
        const int heads = q_heads + (write_cache ? 2 * kv_heads : 0);
        for (int h = 0; h < heads; ++h) {
            const bool is_q = h < q_heads, is_k = !is_q && h < q_heads + kv_heads;
            float ss = 0.f;
            for (int d = 0; d < head_dim; ++d) {
                float value = qkv[r * width + static_cast<long>(h) * head_dim + d];
                for (int p = 1; p < planes; ++p) value += qkv[p * plane + r * width + static_cast<long>(h) * head_dim + d];
                head[d] = value;
                ss = ss + value * value;
            }
            float* dst = nullptr;
            int token = 0;
            if (is_q) {
                dst = q_out + (static_cast<long>(r) * q_heads + h) * head_dim;
            } else {
                const int kvh = is_k ? h - q_heads : h - q_heads - kv_heads;
                const int page = block_table[static_cast<long>(row_entry[r]) * max_blocks + pos / page_tokens];
                if (page < 0) continue;
                dst = (is_k ? k_pool : v_pool) + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
                token = pos % page_tokens;
            }
            if (!is_q && !is_k) {
                for (int d = 0; d < head_dim; ++d) dst[value_offset(token, d, head_dim)] = head[d];
                continue;
            }
            const float* gain = is_q ? q_gain : k_gain;
            if (gain) {
                const float inv = 1.0f / std::sqrt(ss / static_cast<float>(head_dim) + eps);
                for (int d = 0; d < head_dim; ++d) head[d] = (head[d] * gain[d]) * inv;
            }
            if (cos_table) {
                const int tpos = pos < table_positions ? pos : table_positions - 1;
                for (int i = 0; i < half; ++i) {
                    const float c = cos_table[static_cast<long>(tpos) * half + i], s = sin_table[static_cast<long>(tpos) * half + i];
                    const int first = pairing == 0 ? i : 2 * i, second = pairing == 0 ? i + half : 2 * i + 1;
                    const float u = head[first], v = head[second];
                    head[first] = u * c - v * s;
                    head[second] = u * s + v * c;
                }
            }
            for (int d = 0; d < head_dim; ++d) dst[is_q ? d : key_offset(token, d, page_tokens)] = head[d];
        }
    }
    return 0;
}

// Each query row attends the keys of its request from max(0, position - window + 1) (window 0: from 0) to its
// own position: scores in key order, one maximum, weights exp(score - maximum), their sum, then the weighted
// values summed in key order and divided (crates/leone/src/cpu.rs:2299-2357).  A key without a page gives NaN.
int leone_ref_attention(const float* q, float* out, const float* k_pool, const float* v_pool, const int* positions,
                        const int* row_entry, const int* block_table, int max_blocks, int rows, int q_heads,
                        int kv_heads, int head_dim, int page_tokens, float scale, int window) {
    if (!q || !out || !k_pool || !v_pool || !positions || !row_entry || !block_table || rows <= 0 || q_heads <= 0 ||
        kv_heads <= 0 || q_heads % kv_heads || head_dim <= 0 || head_dim % 8 || page_tokens <= 0 || page_tokens % 8 ||
        max_blocks <= 0 || window < 0)
        return LEONE_HOST_INVALID;
    const int group = q_heads / kv_heads;
    std::vector<float> score;
    for (int r = 0; r < rows; ++r) {
        const int n = positions[r] + 1;
        const int lo = (window > 0 && n - window > 0) ? n - window : 0;
        const int* table = block_table + static_cast<long>(row_entry[r]) * max_blocks;
        for (int h = 0; h < q_heads; ++h) {
            const int kvh = h / group;
            const float* qh = q + (static_cast<long>(r) * q_heads + h) * head_dim;
            float* oh = out + (static_cast<long>(r) * q_heads + h) * head_dim;
            score.assign(n - lo, 0.f);
            bool unmapped = false;
            float top = -std::numeric_limits<float>::infinity();
            for (int key = lo; key < n; ++key) {
                const int page = table[key / page_tokens];
                if (page < 0) {
                    unmapped = true;
                    break;
                }
                const float* kp = k_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot = dot + qh[d] * kp[key_offset(key % page_tokens, d, page_tokens)];
                score[key - lo] = dot * scale;
                top = score[key - lo] > top ? score[key - lo] : top;
            }
            if (unmapped) {
                for (int d = 0; d < head_dim; ++d) oh[d] = std::numeric_limits<float>::quiet_NaN();
                continue;
            }
            float total = 0.f;
            for (int key = lo; key < n; ++key) {
                score[key - lo] = std::exp(score[key - lo] - top);
                total = total + score[key - lo];
            }
            for (int d = 0; d < head_dim; ++d) {
                float sum = 0.f;
                for (int key = lo; key < n; ++key) {
                    const int page = table[key / page_tokens];
                    const float* vp = v_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
                    sum = sum + score[key - lo] * vp[value_offset(key % page_tokens, d, head_dim)];
                }
                oh[d] = sum / total;
            }
        }
    }
    return 0;
}

// c[m,n] = a[m,k] . b[n,k]^T, every sum left to right in float.
int leone_ref_gemm(const float* a, const float* b, float* c, int m, int n, int k) {
    if (!a || !b || !c || m <= 0 || n <= 0 || k <= 0) return LEONE_HOST_INVALID;
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float sum = 0.f;
            for (int e = 0; e < k; ++e) sum = sum + a[static_cast<long>(i) * k + e] * b[static_cast<long>(j) * k + e];
            c[static_cast<long>(i) * n + j] = sum;
        }
    return 0;
}

// in [rows, 2 ffn]: every 16 columns are 8 gate values, then their 8 up values; out [rows, ffn] =
// gate / (1 + exp(-gate)) * up (crates/leone/src/cpu.rs:892-907).
int leone_ref_swiglu(const float* gate_up, float* out, int rows, int ffn) {
    if (!gate_up || !out || rows <= 0 || ffn <= 0 || ffn % 8) return LEONE_HOST_INVALID;
    for (long r = 0; r < rows; ++r)
        for (int f = 0; f < ffn; ++f) {
            const float gate = gate_up[r * 2 * ffn + 16 * (f / 8) + f % 8];
            const float up = gate_up[r * 2 * ffn + 16 * (f / 8) + 8 + f % 8];
            out[r * ffn + f] = (gate / (1.0f + std::exp(-gate))) * up;
        }
    return 0;
}

// The highest finite logit of each row, the lowest index on a tie, -1 if there is none
// (crates/leone/src/sampler.rs:787-799).
int leone_ref_argmax(const float* logits, int* out, int rows, int vocab) {
    if (!logits || !out || rows <= 0 || vocab <= 0) return LEONE_HOST_INVALID;
    for (long r = 0; r < rows; ++r) {
        int best = -1;
        for (int i = 0; i < vocab; ++i) {
            const float v = logits[r * vocab + i];
            if (std::isfinite(v) && (best < 0 || v > logits[r * vocab + best])) best = i;
        }
        out[r] = best;
    }
    return 0;
}

// One token a row: weights exp(l / t - max / t) over the finite logits in double, the first token in id order
// whose running share of the total exceeds the uniform value, the last eligible one if rounding leaves none; -1
// for a row without a finite logit (crates/leone/src/sampler.rs:502-534, 843-858).
int leone_ref_sample_temperature(const float* logits, const double* temperature, const double* uniform, int* out,
                                 int rows, int vocab) {
    if (!logits || !temperature || !uniform || !out || rows <= 0 || vocab <= 0) return LEONE_HOST_INVALID;
    for (long r = 0; r < rows; ++r) {
        const float* row = logits + r * vocab;
        if (!(temperature[r] > 0.0)) return LEONE_HOST_INVALID;
        double top = -std::numeric_limits<double>::infinity();
        int last = -1;
        for (int i = 0; i < vocab; ++i)
            if (std::isfinite(row[i])) {
                top = row[i] > top ? row[i] : top;
                last = i;
            }
        out[r] = last;
        if (last < 0) continue;
        double total = 0.0;
        for (int i = 0; i < vocab; ++i)
            if (std::isfinite(row[i])) total += std::exp(row[i] / temperature[r] - top / temperature[r]);
        double running = 0.0;
        for (int i = 0; i < vocab; ++i) {
            if (!std::isfinite(row[i])) continue;
            running += std::exp(row[i] / temperature[r] - top / temperature[r]);
            if (running / total > uniform[r]) {
                out[r] = i;
                break;
            }
        }
    }
    return 0;
}

}  // extern "C"
