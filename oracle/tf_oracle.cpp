// tf_oracle.cpp — CPU restatement of the reference's FP32 validation path.
//
// TEST INFRASTRUCTURE ONLY: see tf_oracle.h.  The product never links this file.
// Build with -ffp-contract=off so that a*b+c is two roundings wherever the
// reference writes two operations; fused operations are spelled fmaf().
#include "tf_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <unordered_set>
#include <vector>

namespace {

inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline uint16_t load_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

constexpr int G = TFO_GROUP_SIZE;
constexpr float kGeluCoeff = 0.7978845608028654f;  // sqrt(2/pi)
constexpr float kGeluCubic = 0.044715f;

inline float gelu_tanh_ref(float xv) {                 // VS/Reference/MoE/Moe.swift:25-27
    const float inner = kGeluCoeff * (xv + kGeluCubic * xv * xv * xv);
    return 0.5f * xv * (1.0f + std::tanh(inner));
}

inline float gelu_tanh_kernel(float x) {               // M/MoE/moe.metal:53-60
    const float x3 = x * x * x;
    float inner = kGeluCoeff * (x + kGeluCubic * x3);
    inner = std::min(std::max(inner, -20.0f), 20.0f);
    return 0.5f * x * (1.0f + std::tanh(inner));
}

inline void dequant4_row(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out) {
    const int groups = n / G;
    for (int g = 0; g < groups; ++g) {
        const float scale = tfo_bf16_to_float(scales[g]);
        const float bias = tfo_bf16_to_float(biases[g]);
        for (int k = 0; k < G; ++k) {
            const uint8_t b = packed[g * (G / 2) + (k / 2)];
            const int nibble = (k & 1) == 0 ? (b & 0x0F) : (b >> 4);
            out[g * G + k] = (float)nibble * scale + bias;
        }
    }
}

inline void dequant8_row(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out) {
    const int groups = n / G;
    for (int g = 0; g < groups; ++g) {
        const float scale = tfo_bf16_to_float(scales[g]);
        const float bias = tfo_bf16_to_float(biases[g]);
        for (int k = 0; k < G; ++k) out[g * G + k] = (float)packed[g * G + k] * scale + bias;
    }
}

inline float dot_f32(const float *a, const float *b, int n) {   // stands in for vDSP_dotpr
    float acc = 0.0f;
    for (int i = 0; i < n; ++i) acc += a[i] * b[i];
    return acc;
}

// One row of an int4 matrix living at byte offsets inside a blob (scales/biases may be 2-aligned only).
inline float blob_row_dot(const uint8_t *blob, uint32_t w_off, uint32_t s_off, uint32_t b_off, int row, int n,
                          const float *x, float *scratch) {
    const int groups = n / G;
    const uint8_t *w = blob + w_off + (int64_t)row * (n / 2);
    const uint8_t *s = blob + s_off + (int64_t)row * groups * 2;
    const uint8_t *b = blob + b_off + (int64_t)row * groups * 2;
    for (int g = 0; g < groups; ++g) {
        const float scale = tfo_bf16_to_float(load_u16(s + 2 * g));
        const float bias = tfo_bf16_to_float(load_u16(b + 2 * g));
        for (int k = 0; k < G; ++k) {
            const uint8_t by = w[g * (G / 2) + (k / 2)];
            const int nibble = (k & 1) == 0 ? (by & 0x0F) : (by >> 4);
            scratch[g * G + k] = (float)nibble * scale + bias;
        }
    }
    return dot_f32(scratch, x, n);
}

// The per-lane arithmetic shared by the reference's one-SIMD-per-row int4 kernels
// (M/Quant/dequant_int4.metal:124-171 == M/MoE/moe.metal:203-247 == M/Sampling/logit.metal:646-690).
// S/B given as byte pointers because blob-resident rows are only 2-byte aligned.
float kernel_row_int4(const uint8_t *w_row, const uint8_t *s_row, const uint8_t *b_row, const uint16_t *x_f16, int n) {
    const int groups = n / G;
    const int full_blocks = groups / 4;
    float lane_acc[32];
    for (int lane = 0; lane < 32; ++lane) {
        float acc = 0.0f;
        for (int blk = 0; blk < full_blocks; ++blk) {
            const int byte_base = blk * 128 + lane * 4;
            const int g = blk * 4 + (lane >> 3);
            const float s = tfo_bf16_to_float(load_u16(s_row + 2 * g));
            const float b = tfo_bf16_to_float(load_u16(b_row + 2 * g));
            const int elem = byte_base * 2;
            float e[8];
            for (int i = 0; i < 8; ++i) e[i] = tfo_f16_to_float(x_f16[elem + i]);
            float dot = 0.0f;
            for (int i = 0; i < 4; ++i) {
                const uint8_t by = w_row[byte_base + i];
                dot = fmaf((float)(by & 0x0F), e[2 * i], dot);
                dot = fmaf((float)(by >> 4), e[2 * i + 1], dot);
            }
            const float sum = e[0] + e[1] + e[2] + e[3] + e[4] + e[5] + e[6] + e[7];
            acc = fmaf(s, dot, acc);
            acc = fmaf(b, sum, acc);
        }
        for (int g = full_blocks * 4; g < groups; ++g) {
            const float s = tfo_bf16_to_float(load_u16(s_row + 2 * g));
            const float b = tfo_bf16_to_float(load_u16(b_row + 2 * g));
            const uint8_t by = w_row[g * (G / 2) + lane];
            const float x0 = tfo_f16_to_float(x_f16[g * G + lane * 2]);
            const float x1 = tfo_f16_to_float(x_f16[g * G + lane * 2 + 1]);
            float dot = fmaf((float)(by & 0x0F), x0, 0.0f);
            dot = fmaf((float)(by >> 4), x1, dot);
            const float sum = x0 + x1;
            acc = fmaf(s, dot, acc);
            acc = fmaf(b, sum, acc);
        }
        lane_acc[lane] = acc;
    }
    float total = 0.0f;   // simd_sum: order unspecified by the reference; lanes taken in order here
    for (int lane = 0; lane < 32; ++lane) total += lane_acc[lane];
    return total;
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------- codecs
uint16_t tfo_bf16_bits(float x) {
    const uint32_t bits = f32_bits(x);
    const uint32_t lsb = (bits >> 16) & 1u;
    const uint32_t rounding_bias = 0x7FFFu + lsb;
    const uint32_t rounded = (bits + rounding_bias) >> 16;   // wraps like Swift's &+
    return (uint16_t)rounded;
}

float tfo_bf16_to_float(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

uint16_t tfo_f16_bits(float f) {
    const uint32_t x = f32_bits(f);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t e = (x >> 23) & 0xFFu;
    uint32_t m = x & 0x7FFFFFu;
    if (e == 0xFFu) {
        if (m == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7C00u | 0x0200u | (m >> 13));
    }
    const int32_t he = (int32_t)e - 112;
    if (he >= 31) return (uint16_t)(sign | 0x7C00u);
    if (he <= 0) {
        if (he < -10) return (uint16_t)sign;
        m |= 0x800000u;
        const int shift = 14 - he;
        uint32_t hm = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t h = sign | ((uint32_t)he << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)h;
}

float tfo_f16_to_float(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        int shift = 0;
        while (!(m & 0x400u)) { m <<= 1; ++shift; }
        m &= 0x3FFu;
        return bits_f32(sign | ((uint32_t)(113 - shift) << 23) | (m << 13));
    }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

// ---------------------------------------------------------------- seeded streams
uint64_t tfo_splitmix64_next(uint64_t *state) {
    *state += 0x9E3779B97F4A7C15ull;
    uint64_t z = *state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

float tfo_splitmix64_uniform(uint64_t *state, float lo, float hi) {
    const float u = (float)(tfo_splitmix64_next(state) >> 40) / (float)(1 << 24);
    return lo + (hi - lo) * u;
}

uint64_t tfo_seedtree_key(uint64_t root, const char *label) {
    uint64_t h = 0xCBF29CE484222325ull;
    for (const unsigned char *p = (const unsigned char *)label; *p; ++p) {
        h ^= (uint64_t)*p;
        h *= 0x100000001B3ull;
    }
    return root ^ h;
}

void tfo_fill_uniform(uint64_t *state, float lo, float hi, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = tfo_splitmix64_uniform(state, lo, hi);
}

// ---------------------------------------------------------------- quantizer
static void quantize_affine(const float *row, int n, int levels, bool nibbles, uint8_t *packed, uint16_t *scales,
                            uint16_t *biases) {
    const int groups = n / G;
    if (nibbles) std::memset(packed, 0, (size_t)n / 2);
    for (int g = 0; g < groups; ++g) {
        float wmin = std::numeric_limits<float>::infinity();
        float wmax = -std::numeric_limits<float>::infinity();
        for (int k = 0; k < G; ++k) {
            const float w = row[g * G + k];
            if (w < wmin) wmin = w;
            if (w > wmax) wmax = w;
        }
        float scale_f, bias_f;
        if (wmax == wmin) { scale_f = 1.0f; bias_f = wmin; }
        else { scale_f = (wmax - wmin) / (float)levels; bias_f = wmin; }
        const uint16_t s_bits = tfo_bf16_bits(scale_f);
        const uint16_t b_bits = tfo_bf16_bits(bias_f);
        scales[g] = s_bits;
        biases[g] = b_bits;
        const float scale = tfo_bf16_to_float(s_bits);
        const float bias = tfo_bf16_to_float(b_bits);
        const float inv_scale = scale == 0.0f ? 0.0f : 1.0f / scale;
        for (int k = 0; k < G; ++k) {
            const float w = row[g * G + k];
            int q = (int)std::round((w - bias) * inv_scale);   // Swift .rounded(): half away from zero
            q = std::max(0, std::min(levels, q));
            if (nibbles) {
                const uint8_t nib = (uint8_t)q & 0x0F;
                const int byte_idx = g * (G / 2) + (k / 2);
                if ((k & 1) == 0) packed[byte_idx] = (uint8_t)((packed[byte_idx] & 0xF0) | nib);
                else packed[byte_idx] = (uint8_t)((packed[byte_idx] & 0x0F) | (nib << 4));
            } else {
                packed[g * G + k] = (uint8_t)q;
            }
        }
    }
}

void tfo_quantize_int4_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    quantize_affine(row, n, 15, true, packed, scales, biases);
}
void tfo_quantize_int8_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    quantize_affine(row, n, 255, false, packed, scales, biases);
}
void tfo_dequantize_int4_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out) {
    dequant4_row(packed, scales, biases, n, out);
}
void tfo_dequantize_int8_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out) {
    dequant8_row(packed, scales, biases, n, out);
}

void tfo_quantize_int4_matrix(const float *w, int m, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    const int groups = n / G;
    for (int r = 0; r < m; ++r)
        tfo_quantize_int4_affine(w + (int64_t)r * n, n, packed + (int64_t)r * (n / 2), scales + (int64_t)r * groups,
                                 biases + (int64_t)r * groups);
}
void tfo_quantize_int8_matrix(const float *w, int m, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    const int groups = n / G;
    for (int r = 0; r < m; ++r)
        tfo_quantize_int8_affine(w + (int64_t)r * n, n, packed + (int64_t)r * n, scales + (int64_t)r * groups,
                                 biases + (int64_t)r * groups);
}
void tfo_dequantize_int4_matrix(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int m, int n, float *out) {
    const int groups = n / G;
    for (int r = 0; r < m; ++r)
        dequant4_row(packed + (int64_t)r * (n / 2), scales + (int64_t)r * groups, biases + (int64_t)r * groups, n,
                     out + (int64_t)r * n);
}
void tfo_dequantize_int8_matrix(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int m, int n, float *out) {
    const int groups = n / G;
    for (int r = 0; r < m; ++r)
        dequant8_row(packed + (int64_t)r * n, scales + (int64_t)r * groups, biases + (int64_t)r * groups, n,
                     out + (int64_t)r * n);
}

// ---------------------------------------------------------------- error metrics
float tfo_rel_error(const float *actual, const float *reference, int64_t n) {
    float max_abs_diff = 0.0f, ref_norm = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        max_abs_diff = std::max(max_abs_diff, std::fabs(actual[i] - reference[i]));
        ref_norm = std::max(ref_norm, std::fabs(reference[i]));
    }
    return max_abs_diff / std::max(ref_norm, 1e-6f);
}
float tfo_max_abs_diff(const float *a, const float *b, int64_t n) {
    float m = 0.0f;
    for (int64_t i = 0; i < n; ++i) m = std::max(m, std::fabs(a[i] - b[i]));
    return m;
}
float tfo_bounded_rel(const float *actual, const float *reference, int64_t n, float abs_floor) {
    float worst = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        const float diff = std::fabs(actual[i] - reference[i]);
        const float denom = std::max(std::fabs(reference[i]), abs_floor);
        worst = std::max(worst, diff / denom);
    }
    return worst;
}

// ---------------------------------------------------------------- GEMV references
void tfo_int4_gemv_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x, float *y, int64_t m,
                       int n, int threads) {
    const int groups = n / G;
#pragma omp parallel num_threads(threads > 1 ? threads : 1) if (threads > 1)
    {
        std::vector<float> w_row((size_t)n);
#pragma omp for schedule(static)
        for (int64_t row = 0; row < m; ++row) {
            dequant4_row(W + row * (n / 2), S + row * groups, B + row * groups, n, w_row.data());
            y[row] = dot_f32(w_row.data(), x, n);
        }
    }
}

void tfo_int8_gemv_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x, float *y, int64_t m,
                       int n, int threads) {
    const int groups = n / G;
#pragma omp parallel num_threads(threads > 1 ? threads : 1) if (threads > 1)
    {
        std::vector<float> w_row((size_t)n);
#pragma omp for schedule(static)
        for (int64_t row = 0; row < m; ++row) {
            dequant8_row(W + row * n, S + row * groups, B + row * groups, n, w_row.data());
            y[row] = dot_f32(w_row.data(), x, n);
        }
    }
}

void tfo_int4_gemv_f64(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x, double *y, int64_t m, int n) {
    const int groups = n / G;
    std::vector<float> w_row((size_t)n);
    for (int64_t row = 0; row < m; ++row) {
        dequant4_row(W + row * (n / 2), S + row * groups, B + row * groups, n, w_row.data());
        double acc = 0.0;
        for (int i = 0; i < n; ++i) acc += (double)w_row[i] * (double)x[i];
        y[row] = acc;
    }
}

void tfo_int8_gemv_f64(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x, double *y, int64_t m, int n) {
    const int groups = n / G;
    std::vector<float> w_row((size_t)n);
    for (int64_t row = 0; row < m; ++row) {
        dequant8_row(W + row * n, S + row * groups, B + row * groups, n, w_row.data());
        double acc = 0.0;
        for (int i = 0; i < n; ++i) acc += (double)w_row[i] * (double)x[i];
        y[row] = acc;
    }
}

// ---------------------------------------------------------------- primitives
void tfo_gelu_tanh(const float *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_tanh_ref(x[i]);
}

void tfo_rmsnorm_ref(const float *x, const float *weight, float eps, float *y, int d) {
    float sum_sq = 0.0f;                       // vDSP_svesq
    for (int i = 0; i < d; ++i) sum_sq += x[i] * x[i];
    const float inv_rms = 1.0f / std::sqrt(sum_sq / (float)d + eps);
    for (int i = 0; i < d; ++i) y[i] = (x[i] * weight[i]) * inv_rms;   // vDSP_vmul then vDSP_vsmul
}

// ---------------------------------------------------------------- MoE references
void tfo_moe_run_ffn(const uint8_t *blob, const tfo_expert_offsets *off, const float *x, float *y, int d, int f) {
    std::vector<float> scratch((size_t)std::max(d, f));
    std::vector<float> act((size_t)f);
    for (int r = 0; r < f; ++r) {
        const float gate = blob_row_dot(blob, off->gate_W_off, off->gate_s_off, off->gate_b_off, r, d, x, scratch.data());
        const float up = blob_row_dot(blob, off->up_W_off, off->up_s_off, off->up_b_off, r, d, x, scratch.data());
        act[r] = gelu_tanh_ref(gate) * up;
    }
    for (int r = 0; r < d; ++r)
        y[r] = blob_row_dot(blob, off->down_W_off, off->down_s_off, off->down_b_off, r, f, act.data(), scratch.data());
}

void tfo_moe_apply_streamed_routed(const uint8_t *const *blobs, const tfo_expert_offsets *off, const float *x,
                                   const float *residual, const float *routing_w, int n_slots, float *y, int d, int f,
                                   int threads) {
    std::vector<float> outs((size_t)n_slots * d);
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) if (threads > 1) schedule(dynamic, 1)
    for (int slot = 0; slot < n_slots; ++slot) tfo_moe_run_ffn(blobs[slot], off, x, outs.data() + (size_t)slot * d, d, f);
    for (int i = 0; i < d; ++i) y[i] = residual[i];
    for (int slot = 0; slot < n_slots; ++slot) {
        const float w = routing_w[slot];
        const float *out = outs.data() + (size_t)slot * d;
        for (int i = 0; i < d; ++i) y[i] = y[i] + out[i] * w;   // vDSP_vsmul then vDSP_vadd
    }
}

void tfo_router_reference(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *hidden,
                          const float *effective_scale, const float *expert_scale, int num_experts, int d, int top_k,
                          uint32_t *out_indices, float *out_weights, float *out_logits) {
    std::vector<float> scaled((size_t)d), logits((size_t)num_experts);
    for (int i = 0; i < d; ++i) scaled[i] = hidden[i] * effective_scale[i];
    tfo_int8_gemv_ref(W, S, B, scaled.data(), logits.data(), num_experts, d, 1);
    if (out_logits) std::memcpy(out_logits, logits.data(), sizeof(float) * (size_t)num_experts);
    std::vector<uint32_t> order((size_t)num_experts);
    for (int e = 0; e < num_experts; ++e) order[e] = (uint32_t)e;
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
        return logits[a] == logits[b] ? a < b : logits[a] > logits[b];
    });
    const int k = std::min(top_k, num_experts);
    const float maximum = k > 0 ? logits[order[0]] : 0.0f;
    std::vector<float> exps((size_t)k);
    float sum = 0.0f;
    for (int i = 0; i < k; ++i) { exps[i] = std::exp(logits[order[i]] - maximum); sum += exps[i]; }
    for (int i = 0; i < k; ++i) {
        out_indices[i] = order[i];
        out_weights[i] = exps[i] / sum * expert_scale[order[i]];
    }
}

void tfo_shared_expert_ref(const uint8_t *gW, const uint16_t *gS, const uint16_t *gB, const uint8_t *uW,
                           const uint16_t *uS, const uint16_t *uB, const uint8_t *dW, const uint16_t *dS,
                           const uint16_t *dB, const float *x, float *y, int d, int f, int threads) {
    std::vector<float> gate((size_t)f), up((size_t)f), act((size_t)f);
    tfo_int4_gemv_ref(gW, gS, gB, x, gate.data(), f, d, threads);
    tfo_int4_gemv_ref(uW, uS, uB, x, up.data(), f, d, threads);
    for (int i = 0; i < f; ++i) {
        const float g = gate[i];
        const float cube = g * g * g;
        const double inner = 0.7978845608028654 * (double)(g + 0.044715f * cube);
        const float gelu = (float)(0.5 * (double)g * (1.0 + std::tanh(inner)));
        act[i] = tfo_f16_to_float(tfo_f16_bits(gelu * up[i]));
    }
    tfo_int4_gemv_ref(dW, dS, dB, act.data(), y, d, f, threads);
}

// ---------------------------------------------------------------- lm_head
uint32_t tfo_lm_head_cpu_greedy(const uint16_t *hidden_f16, const uint16_t *norm_w_bf16, const uint8_t *W,
                                const uint16_t *S, const uint16_t *B, int d, int64_t v, float eps, float *logits_out,
                                int threads) {
    std::vector<float> hidden((size_t)d), norm_w((size_t)d), normed((size_t)d);
    for (int i = 0; i < d; ++i) { hidden[i] = tfo_f16_to_float(hidden_f16[i]); norm_w[i] = tfo_bf16_to_float(norm_w_bf16[i]); }
    tfo_rmsnorm_ref(hidden.data(), norm_w.data(), eps, normed.data(), d);
    for (int i = 0; i < d; ++i) normed[i] = tfo_f16_to_float(tfo_f16_bits(normed[i]));

    std::vector<float> local;
    float *logits = logits_out;
    if (!logits) { local.resize((size_t)v); logits = local.data(); }
    tfo_int4_gemv_ref(W, S, B, normed.data(), logits, v, d, threads);
    float best_value = -std::numeric_limits<float>::infinity();
    uint32_t best_index = 0;
    for (int64_t row = 0; row < v; ++row) {
        if (logits[row] > best_value) { best_value = logits[row]; best_index = (uint32_t)row; }
    }
    return best_index;
}

// ---------------------------------------------------------------- prefill
void tfo_prefill_make_pairs(const uint32_t *indices, const uint16_t *weights_f16, int query_count, int top_k, tfo_pair *pairs) {
    for (int token = 0; token < query_count; ++token)
        for (int rank = 0; rank < top_k; ++rank) {
            const int i = token * top_k + rank;
            pairs[i] = tfo_pair{(uint32_t)token, indices[i], (uint32_t)rank, (uint32_t)weights_f16[i]};
        }
}

int tfo_prefill_group_pairs(const tfo_pair *pairs, int64_t pair_count, int query_count, int top_k, int num_experts,
                            int tile_expert_count, const uint64_t *expert_sort_keys, int sort_key_count,
                            tfo_pair *sorted_pairs, uint32_t *per_expert_offsets, uint32_t *per_expert_counts,
                            tfo_group *groups, int *n_groups, tfo_tile *tiles, int *n_tiles) {
    if (query_count < 0) return TFO_GROUP_INVALID_QUERY_COUNT;
    if (top_k <= 0) return TFO_GROUP_INVALID_TOP_K;
    if (num_experts <= 0) return TFO_GROUP_INVALID_NUM_EXPERTS;
    if (tile_expert_count < 1 || tile_expert_count > 16) return TFO_GROUP_INVALID_TILE_EXPERT_COUNT;
    if (expert_sort_keys && sort_key_count != num_experts) return TFO_GROUP_SORT_KEY_COUNT_MISMATCH;
    if (pair_count != (int64_t)query_count * top_k) return TFO_GROUP_PAIR_COUNT_MISMATCH;

    std::unordered_set<uint64_t> seen;
    seen.reserve((size_t)pair_count);
    for (int64_t i = 0; i < pair_count; ++i) {
        const tfo_pair &p = pairs[i];
        if (!(p.token < (uint32_t)query_count)) return TFO_GROUP_TOKEN_OUT_OF_RANGE;
        if (!(p.rank < (uint32_t)top_k)) return TFO_GROUP_RANK_OUT_OF_RANGE;
        if (!(p.expert < (uint32_t)num_experts)) return TFO_GROUP_EXPERT_OUT_OF_RANGE;
        const uint64_t key = ((uint64_t)p.token << 32) | (uint64_t)p.rank;
        if (!seen.insert(key).second) return TFO_GROUP_DUPLICATE_TOKEN_RANK;
    }

    std::vector<tfo_pair> sorted(pairs, pairs + pair_count);
    std::stable_sort(sorted.begin(), sorted.end(), [&](const tfo_pair &a, const tfo_pair &b) {
        if (expert_sort_keys) {
            const uint64_t ka = expert_sort_keys[a.expert], kb = expert_sort_keys[b.expert];
            if (ka != kb) return ka < kb;
        }
        if (a.expert != b.expert) return a.expert < b.expert;
        if (a.token != b.token) return a.token < b.token;
        return a.rank < b.rank;
    });
    for (int e = 0; e < num_experts; ++e) { per_expert_offsets[e] = 0xFFFFFFFFu; per_expert_counts[e] = 0; }
    int ng = 0;
    int64_t i = 0;
    while (i < pair_count) {
        const uint32_t expert = sorted[(size_t)i].expert;
        const int64_t start = i;
        while (i < pair_count && sorted[(size_t)i].expert == expert) ++i;
        per_expert_offsets[expert] = (uint32_t)start;
        per_expert_counts[expert] = (uint32_t)(i - start);
        groups[ng++] = tfo_group{expert, (uint32_t)start, (uint32_t)(i - start)};
    }
    int nt = 0;
    int group_start = 0;
    while (group_start < ng) {
        const int group_end = std::min(ng, group_start + tile_expert_count);
        const tfo_group &first = groups[group_start];
        const tfo_group &last = groups[group_end - 1];
        const uint32_t pair_end = last.pair_start + last.pair_count;
        tiles[nt++] = tfo_tile{(uint32_t)group_start, (uint32_t)(group_end - group_start), first.pair_start,
                               pair_end - first.pair_start};
        group_start = group_end;
    }
    std::copy(sorted.begin(), sorted.end(), sorted_pairs);
    *n_groups = ng;
    *n_tiles = nt;
    return TFO_GROUP_OK;
}

float tfo_prefill_cpu_int4_dot(const uint8_t *bytes, int64_t base, int64_t w_off, int64_t s_off, int64_t b_off, int row,
                               int n, const float *x) {
    const int groups = n / G;
    const int row_bytes = n / 2;
    const int64_t w_row = base + w_off + (int64_t)row * row_bytes;
    const int64_t s_row = base + s_off + (int64_t)row * groups * 2;
    const int64_t b_row = base + b_off + (int64_t)row * groups * 2;
    float acc = 0.0f;
    for (int group = 0; group < groups; ++group) {
        const float scale = tfo_bf16_to_float(load_u16(bytes + s_row + group * 2));
        const float bias = tfo_bf16_to_float(load_u16(bytes + b_row + group * 2));
        for (int k = 0; k < G; ++k) {
            const int col = group * G + k;
            const uint8_t packed = bytes[w_row + col / 2];
            const float q = (k & 1) == 0 ? (float)(packed & 0x0F) : (float)(packed >> 4);
            acc += (q * scale + bias) * x[col];
        }
    }
    return acc;
}

void tfo_prefill_route_partials(const tfo_pair *sorted_pairs, int64_t pair_count, int query_count,
                                const uint16_t *hidden_f16, int hidden_stride, const uint8_t *pool, int64_t pool_stride,
                                const tfo_expert_offsets *off, int top_k, int d, int f, uint16_t fill_f16,
                                uint16_t *out_f16, int threads) {
    const int64_t total = (int64_t)query_count * top_k * d;
    for (int64_t i = 0; i < total; ++i) out_f16[i] = fill_f16;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) if (threads > 1) schedule(dynamic, 4)
    for (int64_t p = 0; p < pair_count; ++p) {
        const tfo_pair &pair = sorted_pairs[p];
        const int64_t expert_base = (int64_t)pair.expert * pool_stride;
        const int64_t x_base = (int64_t)pair.token * hidden_stride;
        std::vector<float> x((size_t)d), act((size_t)f);
        for (int i = 0; i < d; ++i) x[i] = tfo_f16_to_float(hidden_f16[x_base + i]);
        for (int row = 0; row < f; ++row) {
            const float gate = tfo_prefill_cpu_int4_dot(pool, expert_base, off->gate_W_off, off->gate_s_off, off->gate_b_off, row, d, x.data());
            const float up = tfo_prefill_cpu_int4_dot(pool, expert_base, off->up_W_off, off->up_s_off, off->up_b_off, row, d, x.data());
            act[row] = tfo_f16_to_float(tfo_f16_bits(gelu_tanh_ref(gate) * up));
        }
        const int64_t out_base = ((int64_t)pair.token * top_k + pair.rank) * d;
        for (int row = 0; row < d; ++row) {
            const float value = tfo_prefill_cpu_int4_dot(pool, expert_base, off->down_W_off, off->down_s_off, off->down_b_off, row, f, act.data());
            out_f16[out_base + row] = tfo_f16_bits(value);
        }
    }
}

void tfo_prefill_reduce_token_major(const uint16_t *partials_f16, const uint16_t *weights_f16, int rows, int top_k, int d,
                                    uint16_t *out_f16) {
    for (int token = 0; token < rows; ++token)
        for (int column = 0; column < d; ++column) {
            float accumulator = 0.0f;
            for (int rank = 0; rank < top_k; ++rank) {
                const int64_t partial_index = ((int64_t)token * top_k + rank) * d + column;
                accumulator += tfo_f16_to_float(weights_f16[token * top_k + rank]) * tfo_f16_to_float(partials_f16[partial_index]);
            }
            out_f16[(int64_t)token * d + column] = tfo_f16_bits(accumulator);
        }
}

void tfo_qmm_cpu_reference(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16, int m, int n,
                           int k, float *out, int threads) {
    const int groups = k / G;
    const int row_bytes = k / 2;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) if (threads > 1) schedule(static)
    for (int token = 0; token < m; ++token) {
        std::vector<float> xr((size_t)k);
        for (int c = 0; c < k; ++c) xr[c] = tfo_f16_to_float(x_f16[(int64_t)token * k + c]);
        for (int row = 0; row < n; ++row) {
            float accumulator = 0.0f;
            for (int group = 0; group < groups; ++group) {
                const float scale = tfo_bf16_to_float(S[(int64_t)row * groups + group]);
                const float bias = tfo_bf16_to_float(B[(int64_t)row * groups + group]);
                for (int local_k = 0; local_k < G; ++local_k) {
                    const int column = group * G + local_k;
                    const uint8_t byte = W[(int64_t)row * row_bytes + column / 2];
                    const uint8_t q = (column % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
                    const float weight = (float)q * scale + bias;
                    accumulator = fmaf(weight, xr[column], accumulator);
                }
            }
            out[(int64_t)token * n + row] = tfo_f16_to_float(tfo_f16_bits(accumulator));
        }
    }
}

// ---------------------------------------------------------------- kernel-order restatements
void tfo_k_int4_gemv(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16, float *y_f32, int64_t m, int n) {
    const int groups = n / G;
    for (int64_t row = 0; row < m; ++row)
        y_f32[row] = kernel_row_int4(W + row * (n / 2), (const uint8_t *)(S + row * groups), (const uint8_t *)(B + row * groups), x_f16, n);
}

void tfo_k_router_logits(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *hidden_f16,
                         const uint16_t *eff_scale_bf16, float *logits, int num_experts, int d) {
    const int groups = d / G;
    for (int e = 0; e < num_experts; ++e) {
        const uint8_t *w_row = W + (int64_t)e * d;
        float total = 0.0f;
        for (int lane = 0; lane < 32; ++lane) {
            float acc = 0.0f;
            for (int g = 0; g < groups; ++g) {
                const float s = tfo_bf16_to_float(S[e * groups + g]);
                const float b = tfo_bf16_to_float(B[e * groups + g]);
                const int idx = g * G + lane * 2;
                const float q0 = (float)w_row[idx], q1 = (float)w_row[idx + 1];
                const float x0 = tfo_f16_to_float(hidden_f16[idx]) * tfo_bf16_to_float(eff_scale_bf16[idx]);
                const float x1 = tfo_f16_to_float(hidden_f16[idx + 1]) * tfo_bf16_to_float(eff_scale_bf16[idx + 1]);
                acc = fmaf(s, q0 * x0 + q1 * x1, acc);
                acc = fmaf(b, x0 + x1, acc);
            }
            total += acc;
        }
        logits[e] = total;
    }
}

void tfo_k_router_topk(const float *logits, const uint16_t *per_expert_scale_bf16, int num_experts, int top_k,
                       uint32_t *out_indices, uint16_t *out_weights_f16) {
    const int KK = std::min(top_k, 64);
    uint32_t top_idx[64];
    float top_score[64];
    for (int i = 0; i < 64; ++i) { top_idx[i] = 0; top_score[i] = -std::numeric_limits<float>::infinity(); }
    for (int e = 0; e < num_experts; ++e) {
        const float s = logits[e];
        if (KK > 0 && s <= top_score[KK - 1]) continue;
        int pos = KK;
        for (int i = 0; i < KK; ++i)
            if (s > top_score[i] || (s == top_score[i] && (uint32_t)e < top_idx[i])) { pos = i; break; }
        if (pos >= KK) continue;
        for (int i = KK - 1; i > pos; --i) { top_idx[i] = top_idx[i - 1]; top_score[i] = top_score[i - 1]; }
        top_idx[pos] = (uint32_t)e;
        top_score[pos] = s;
    }
    const float max_s = top_score[0];
    float sum_exp = 0.0f;
    float exps[64];
    for (int i = 0; i < KK; ++i) { exps[i] = std::exp(top_score[i] - max_s); sum_exp += exps[i]; }
    for (int i = 0; i < KK; ++i) {
        const uint32_t expert_idx = top_idx[i];
        const float weight = exps[i] / sum_exp;
        out_indices[i] = expert_idx;
        out_weights_f16[i] = tfo_f16_bits(weight * tfo_bf16_to_float(per_expert_scale_bf16[expert_idx]));
    }
}

void tfo_k_moe_phase1(const uint8_t *const *blobs, const tfo_expert_offsets *off, const uint16_t *x_f16,
                      uint16_t *acts_f16, int d, int f, int top_k) {
    const int groups = d / G;
    for (int slot = 0; slot < top_k; ++slot) {
        const uint8_t *base = blobs[slot];
        for (int r = 0; r < f; ++r) {
            const float g = kernel_row_int4(base + off->gate_W_off + (int64_t)r * (d / 2), base + off->gate_s_off + (int64_t)r * groups * 2,
                                            base + off->gate_b_off + (int64_t)r * groups * 2, x_f16, d);
            const float u = kernel_row_int4(base + off->up_W_off + (int64_t)r * (d / 2), base + off->up_s_off + (int64_t)r * groups * 2,
                                            base + off->up_b_off + (int64_t)r * groups * 2, x_f16, d);
            acts_f16[slot * f + r] = tfo_f16_bits(gelu_tanh_kernel(g) * u);
        }
    }
}

void tfo_k_moe_phase2(const uint8_t *const *blobs, const tfo_expert_offsets *off, const uint16_t *acts_f16,
                      const uint16_t *routing_w_f16, const uint16_t *residual_f16, uint16_t *y_f16, int d, int f) {
    const int groups = f / G;
    for (int row = 0; row < d; ++row) {
        float acc = tfo_f16_to_float(residual_f16[row]);
        for (int s = 0; s < 8; ++s) {
            const uint8_t *base = blobs[s];
            const float value = kernel_row_int4(base + off->down_W_off + (int64_t)row * (f / 2), base + off->down_s_off + (int64_t)row * groups * 2,
                                                base + off->down_b_off + (int64_t)row * groups * 2, acts_f16 + (int64_t)s * f, f);
            acc += tfo_f16_to_float(routing_w_f16[s]) * value;
        }
        y_f16[row] = tfo_f16_bits(acc);
    }
}

void tfo_k_gelu_mul_fp16(const uint16_t *gate_f16, const uint16_t *up_f16, uint16_t *out_f16, int n) {
    for (int i = 0; i < n; ++i)
        out_f16[i] = tfo_f16_bits(gelu_tanh_kernel(tfo_f16_to_float(gate_f16[i])) * tfo_f16_to_float(up_f16[i]));
}

void tfo_k_rmsnorm_bf16w(const uint16_t *x_f16, const uint16_t *w_bf16, float eps, uint16_t *out_f16, int d) {
    float partial[256];
    for (int lid = 0; lid < 256; ++lid) {
        float acc = 0.0f;
        for (int i = lid; i < d; i += 256) { const float v = tfo_f16_to_float(x_f16[i]); acc = fmaf(v, v, acc); }
        partial[lid] = acc;
    }
    float total = 0.0f;
    for (int sg = 0; sg < 8; ++sg) {
        float s = 0.0f;
        for (int lane = 0; lane < 32; ++lane) s += partial[sg * 32 + lane];
        total += s;
    }
    const float inv = 1.0f / std::sqrt(total / (float)d + eps);
    for (int i = 0; i < d; ++i)
        out_f16[i] = tfo_f16_bits(tfo_f16_to_float(x_f16[i]) * inv * tfo_bf16_to_float(w_bf16[i]));
}

// Kernel-order restatement of the row-grid norms: rmsnorm_no_scale / rmsnorm_*_perhead (M/Primitives/rmsnorm.metal:100-175)
// and their prefill twins (M/Prefill/prefill.metal:86-176): head h of token t at t * token_stride + h * d, each row
// normalised on its own exactly as tfo_k_rmsnorm_bf16w does; w_bf16 == nullptr: no scale.  Elements between rows keep
// what out_f16 held.
void tfo_k_rmsnorm_rows(const uint16_t *x_f16, const uint16_t *w_bf16, float eps, uint16_t *out_f16, int tokens, int heads, int d,
                        int token_stride) {
    std::vector<uint16_t> ones;
    for (int t = 0; t < tokens; ++t)
        for (int h = 0; h < heads; ++h) {
            const size_t at = (size_t)t * token_stride + (size_t)h * d;
            if (w_bf16) {
                tfo_k_rmsnorm_bf16w(x_f16 + at, w_bf16, eps, out_f16 + at, d);
            } else {
                // x * inv * 1.0f is x * inv: the weighted routine with unit weights is the unweighted one
                if (ones.empty()) ones.assign((size_t)d, (uint16_t)0x3F80);
                tfo_k_rmsnorm_bf16w(x_f16 + at, ones.data(), eps, out_f16 + at, d);
            }
        }
}

// ---- neighbours of the output head ---------------------------------------------------------------------------------
// VS/Reference/Quant/EmbedLookup.swift:41-68 (applyInt4): one row of the tied int4 table, dequantized and scaled.
void tfo_embed_lookup_int4(const uint8_t *table, const uint16_t *S, const uint16_t *B, uint32_t token, int d, float out_scale, float *out) {
    const int groups = d / G;
    const uint8_t *row = table + (size_t)token * (d / 2);
    for (int i = 0; i < d; ++i) {
        const uint8_t byte = row[i >> 1];
        const int q = (i & 1) == 0 ? (byte & 0x0F) : (byte >> 4);
        const float s = tfo_bf16_to_float(S[(size_t)token * groups + i / G]);
        const float b = tfo_bf16_to_float(B[(size_t)token * groups + i / G]);
        out[i] = ((float)q * s + b) * out_scale;
    }
}

// VS/Reference/Sampling/LogitSoftcapSoftmax.swift:12-48: softcap * tanh(x / softcap), then a two-pass safe softmax.
void tfo_logit_softcap_softmax_ref(const float *x, int v, float softcap, float *out) {
    const float inv_c = 1.0f / softcap;
    float mx = -INFINITY;
    for (int i = 0; i < v; ++i) {
        out[i] = softcap * std::tanh(x[i] * inv_c);
        mx = out[i] > mx ? out[i] : mx;
    }
    float sum = 0.0f;
    for (int i = 0; i < v; ++i) {
        out[i] = std::exp(out[i] - mx);
        sum += out[i];
    }
    const float inv_sum = 1.0f / sum;
    for (int i = 0; i < v; ++i) out[i] *= inv_sum;
}

// M/Sampling/logit.metal:148-181: the sampler's two generators.
static uint64_t sampler_xorshift64(uint64_t &s) {
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s * 2685821657736338717ULL;
}
static float sampler_uniform01(uint64_t &s) { return (float)(uint32_t)(sampler_xorshift64(s) >> 40) * (1.0f / 16777216.0f); }
uint64_t tfo_sampler_xorshift64(uint64_t *state) { return sampler_xorshift64(*state); }
float tfo_sampler_gumbel(uint64_t seed, uint32_t position, uint32_t row) {
    uint64_t x = seed ^ ((uint64_t)position * 0xD2B74407B1CE6E93ull) ^ (uint64_t)row;
    x = x + 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x = x ^ (x >> 31);
    const float u = ((float)(uint32_t)(x >> 40) + 0.5f) * (1.0f / 16777216.0f);
    return -std::log(-std::log(u));
}

// Tail of the truncating sampler, shared by `sample` (M/Sampling/logit.metal:381-447) and `sample_topk64_final` (:566-606):
// values/indices = the k best (probability descending, index ascending).  Returns the token.
static uint32_t sampler_finish(std::vector<float> &values, const std::vector<uint32_t> &indices, uint32_t v, float temperature,
                               float top_p, uint64_t seed) {
    uint32_t kept = 0;
    while (kept < values.size() && indices[kept] < v && std::isfinite(values[kept])) ++kept;
    if (top_p > 0.0f && top_p < 1.0f) {
        float cum = 0.0f;
        uint32_t cut = kept;
        for (uint32_t i = 0; i < kept; ++i) {
            cum += values[i];
            if (cum >= top_p) { cut = i + 1; break; }
        }
        kept = cut;
    }
    const float inv_temp = 1.0f / temperature;
    if (temperature != 1.0f)
        for (uint32_t i = 0; i < kept; ++i) values[i] = std::pow(values[i], inv_temp);
    float surviving = 0.0f;
    for (uint32_t i = 0; i < kept; ++i) surviving += values[i];
    uint64_t rng = seed;
    (void)sampler_xorshift64(rng);
    const float u = sampler_uniform01(rng) * surviving;
    float run = 0.0f;
    uint32_t picked = indices.empty() ? 0u : indices[0];
    for (uint32_t i = 0; i < kept; ++i) {
        run += values[i];
        if (u <= run) { picked = indices[i]; break; }
    }
    return picked;
}

static void sampler_top(const uint16_t *probs_f16, uint32_t v, uint32_t k, std::vector<float> &values, std::vector<uint32_t> &indices) {
    // k rounds of "largest not yet taken, lowest index on ties" == the first k of a stable sort by descending value;
    // NaN never compares greater, so it is never taken (the slot then holds -inf / 0xFFFFFFFF, as in the kernel)
    std::vector<uint32_t> order;
    order.reserve(v);
    for (uint32_t i = 0; i < v; ++i) {
        const float p = tfo_f16_to_float(probs_f16[i]);
        if (p > -INFINITY) order.push_back(i);
    }
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) { return tfo_f16_to_float(probs_f16[a]) > tfo_f16_to_float(probs_f16[b]); });
    values.assign(k, -INFINITY);
    indices.assign(k, 0xFFFFFFFFu);
    for (uint32_t i = 0; i < k && i < order.size(); ++i) {
        values[i] = tfo_f16_to_float(probs_f16[order[i]]);
        indices[i] = order[i];
    }
}

// M/Sampling/logit.metal:183-447 (`sample`): greedy, Gumbel-max, or top-k / top-p / temperature / inverse CDF.
uint32_t tfo_sample(const uint16_t *probs_f16, uint32_t v, float temperature, uint32_t top_k, float top_p, uint64_t seed, uint32_t position) {
    if (temperature <= 0.0f) {
        float best = -INFINITY;
        uint32_t idx = 0u;   // nothing above -inf: every thread of the kernel keeps its initial index 0
        for (uint32_t i = 0; i < v; ++i) {
            const float p = tfo_f16_to_float(probs_f16[i]);
            if (p > best) { best = p; idx = i; }
        }
        return idx;
    }
    if (top_k == 0u && (top_p <= 0.0f || top_p >= 1.0f)) {
        const float inv_t = 1.0f / temperature;
        float best = -INFINITY;
        uint32_t idx = 0xFFFFFFFFu;
        for (uint32_t i = 0; i < v; ++i) {
            const float p = tfo_f16_to_float(probs_f16[i]);
            if (!(p > 0.0f)) continue;
            const float sc = inv_t * std::log(p) + tfo_sampler_gumbel(seed, position, i);
            if (sc > best) { best = sc; idx = i; }
        }
        return idx == 0xFFFFFFFFu ? 0u : idx;
    }
    uint32_t k = top_k == 0u ? v : top_k;
    k = k < 256u ? k : 256u;
    k = k < v ? k : v;
    std::vector<float> values;
    std::vector<uint32_t> indices;
    sampler_top(probs_f16, v, k, values, indices);
    return sampler_finish(values, indices, v, temperature, top_p, seed);
}

// M/Sampling/logit.metal:449-606 + Kernels/Sampling/LogitOutput.swift:88-206 (SampleTopK64): the 64 best through sorted
// 1024-entry tiles, then the same tail.  Tile sorting keeps exactly the 64 best by (value descending, index ascending).
uint32_t tfo_sample_topk64(const uint16_t *probs_f16, uint32_t v, float temperature, float top_p, uint64_t seed) {
    std::vector<float> values;
    std::vector<uint32_t> indices;
    sampler_top(probs_f16, v, 64u < v ? 64u : v, values, indices);
    values.resize(64, -INFINITY);
    indices.resize(64, 0xFFFFFFFFu);
    return sampler_finish(values, indices, 0xFFFFFFFFu, temperature, top_p, seed);
}

// Sum of squares of d fp16 values in the order of the reference's 256-thread, 32-lane two-stage reduction
// (M/Fusions/fused.metal:217-235): strided per-thread fma chains, lane sums, then the per-group partials.
static float k_block_sum_squares(const uint16_t *x_f16, int d) {
    float partial[256];
    for (int lid = 0; lid < 256; ++lid) {
        float acc = 0.0f;
        for (int i = lid; i < d; i += 256) { const float v = tfo_f16_to_float(x_f16[i]); acc = fmaf(v, v, acc); }
        partial[lid] = acc;
    }
    float total = 0.0f;
    for (int sg = 0; sg < 8; ++sg) {
        float s = 0.0f;
        for (int lane = 0; lane < 32; ++lane) s += partial[sg * 32 + lane];
        total += s;
    }
    return total;
}

// M/Fusions/fused.metal:190-269 (fused_post_attn_setup) and its per-row twin M/Prefill/prefill.metal:178-253:
// hidden += rmsnorm(attn, w_post_attn) rounded to fp16 at each stage; then the three views of rmsnorm(hidden).
void tfo_k_post_attn_setup(uint16_t *hidden_f16, const uint16_t *attn_f16, const uint16_t *w_post_attn_bf16,
                           const uint16_t *w_pre_ffn_bf16, const uint16_t *w_pre_ffn2_bf16, float eps, uint16_t *dense_f16,
                           uint16_t *routed_f16, uint16_t *router_f16, int d) {
    const float attn_inv = 1.0f / std::sqrt(k_block_sum_squares(attn_f16, d) / (float)d + eps);
    for (int i = 0; i < d; ++i) {
        const uint16_t an = tfo_f16_bits(tfo_f16_to_float(attn_f16[i]) * attn_inv * tfo_bf16_to_float(w_post_attn_bf16[i]));
        hidden_f16[i] = tfo_f16_bits(tfo_f16_to_float(hidden_f16[i]) + tfo_f16_to_float(an));
    }
    const float hidden_inv = 1.0f / std::sqrt(k_block_sum_squares(hidden_f16, d) / (float)d + eps);
    for (int i = 0; i < d; ++i) {
        const float h = tfo_f16_to_float(hidden_f16[i]) * hidden_inv;
        dense_f16[i] = tfo_f16_bits(h * tfo_bf16_to_float(w_pre_ffn_bf16[i]));
        routed_f16[i] = tfo_f16_bits(h * tfo_bf16_to_float(w_pre_ffn2_bf16[i]));
        router_f16[i] = tfo_f16_bits(h);
    }
}

// M/Fusions/fused.metal:271-375 (fused_layer_tail) and M/Prefill/prefill.metal:255-334:
// hidden = half(half(hidden + rmsnorm(h1 + rmsnorm(h2, w_postffn2), w_postffn)) * half(layer_scalar)), fp16 at every stage.
void tfo_k_layer_tail(const uint16_t *h2_f16, const uint16_t *h1_f16, uint16_t *hidden_f16, const uint16_t *w_postffn2_bf16,
                      const uint16_t *w_postffn_bf16, float eps, float layer_scalar, int d) {
    std::vector<uint16_t> h12(d);
    const float inv_h2 = 1.0f / std::sqrt(k_block_sum_squares(h2_f16, d) / (float)d + eps);
    for (int i = 0; i < d; ++i) {
        const uint16_t t = tfo_f16_bits(tfo_f16_to_float(h2_f16[i]) * inv_h2 * tfo_bf16_to_float(w_postffn2_bf16[i]));
        h12[i] = tfo_f16_bits(tfo_f16_to_float(h1_f16[i]) + tfo_f16_to_float(t));
    }
    const float inv_h12 = 1.0f / std::sqrt(k_block_sum_squares(h12.data(), d) / (float)d + eps);
    const float scale = tfo_f16_to_float(tfo_f16_bits(layer_scalar));
    for (int i = 0; i < d; ++i) {
        const uint16_t t = tfo_f16_bits(tfo_f16_to_float(h12[i]) * inv_h12 * tfo_bf16_to_float(w_postffn_bf16[i]));
        const uint16_t sum = tfo_f16_bits(tfo_f16_to_float(hidden_f16[i]) + tfo_f16_to_float(t));
        hidden_f16[i] = tfo_f16_bits(tfo_f16_to_float(sum) * scale);
    }
}

// T/Core/Kernels/Fusions/FusedLayerTailTests.swift:76-92 (cpuReference): the same chain through the fp32 RmsNorm reference.
void tfo_layer_tail_ref(const uint16_t *h2_f16, const uint16_t *h1_f16, const uint16_t *hidden_f16, const uint16_t *w_postffn2_bf16,
                        const uint16_t *w_postffn_bf16, float eps, float layer_scalar, float *out, int d) {
    std::vector<float> x(d), w2(d), w(d), n(d), h12(d);
    for (int i = 0; i < d; ++i) {
        x[i] = tfo_f16_to_float(h2_f16[i]);
        w2[i] = tfo_bf16_to_float(w_postffn2_bf16[i]);
        w[i] = tfo_bf16_to_float(w_postffn_bf16[i]);
    }
    tfo_rmsnorm_ref(x.data(), w2.data(), eps, n.data(), d);
    for (int i = 0; i < d; ++i)
        h12[i] = tfo_f16_to_float(tfo_f16_bits(tfo_f16_to_float(h1_f16[i]) + tfo_f16_to_float(tfo_f16_bits(n[i]))));
    tfo_rmsnorm_ref(h12.data(), w.data(), eps, n.data(), d);
    const float scale = tfo_f16_to_float(tfo_f16_bits(layer_scalar));
    for (int i = 0; i < d; ++i) {
        const float sum = tfo_f16_to_float(tfo_f16_bits(tfo_f16_to_float(hidden_f16[i]) + tfo_f16_to_float(tfo_f16_bits(n[i]))));
        out[i] = tfo_f16_to_float(tfo_f16_bits(sum * scale));
    }
}

void tfo_k_prefill_router_logits(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *hidden_f16,
                                 const uint16_t *eff_scale_bf16, float *logits, int num_experts, int d) {
    const int groups = d / G;
    for (int e = 0; e < num_experts; ++e) {
        float acc = 0.0f;
        for (int g = 0; g < groups; ++g) {
            const float s = tfo_bf16_to_float(S[e * groups + g]);
            const float b = tfo_bf16_to_float(B[e * groups + g]);
            float dot_qx = 0.0f, sum_x = 0.0f;
            for (int k = 0; k < G; ++k) {
                const int idx = g * G + k;
                const float q = (float)W[(int64_t)e * d + idx];
                const float xv = tfo_f16_to_float(hidden_f16[idx]) * tfo_bf16_to_float(eff_scale_bf16[idx]);
                dot_qx = fmaf(q, xv, dot_qx);
                sum_x += xv;
            }
            acc = fmaf(s, dot_qx, acc);
            acc = fmaf(b, sum_x, acc);
        }
        logits[e] = acc;
    }
}

float tfo_k_prefill_int4_row(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16, int row, int n) {
    const int groups = n / G;
    const uint8_t *w_row = W + (int64_t)row * (n / 2);
    const uint8_t *s_row = (const uint8_t *)S + (int64_t)row * groups * 2;
    const uint8_t *b_row = (const uint8_t *)B + (int64_t)row * groups * 2;
    float acc = 0.0f;
    for (int g = 0; g < groups; ++g) {
        const float scale = tfo_bf16_to_float(load_u16(s_row + 2 * g));
        const float bias = tfo_bf16_to_float(load_u16(b_row + 2 * g));
        float dot_qx = 0.0f, sum_x = 0.0f;
        for (int k = 0; k < G / 2; ++k) {
            const uint8_t packed = w_row[g * (G / 2) + k];
            const float x0 = tfo_f16_to_float(x_f16[g * G + 2 * k]);
            const float x1 = tfo_f16_to_float(x_f16[g * G + 2 * k + 1]);
            dot_qx = fmaf((float)(packed & 0x0F), x0, dot_qx);
            dot_qx = fmaf((float)(packed >> 4), x1, dot_qx);
            sum_x += x0 + x1;
        }
        acc = fmaf(scale, dot_qx, acc);
        acc = fmaf(bias, sum_x, acc);
    }
    return acc;
}

// ---------------------------------------------------------------------------------------------------- attention (decode)
// V/Support/Reference/Attention/Attention.swift:14-108 (AttentionRef.apply): per query head all scores of the window
// [kv_start, seq_len), a stable softmax, then the probability-weighted sum of V.  q [num_q_heads, head_dim] fp32;
// k, v [seq_len, num_kv_heads, head_dim] fp32; window < 0: none; scale <= 0: 1/sqrt(head_dim).  Accumulation in double
// (the reference sums in fp32 through vDSP, whose order is not specified).
void tfo_attention_ref(const float *q, const float *k, const float *v, int head_dim, int num_q_heads, int num_kv_heads, int seq_len,
                       int window, float scale, float *out) {
    const int group = num_q_heads / num_kv_heads;
    const double sc = scale > 0.0f ? (double)scale : 1.0 / std::sqrt((double)head_dim);
    const int kv_start = (window >= 0 && seq_len > window) ? seq_len - window : 0;
    std::vector<double> scores((size_t)std::max(1, seq_len - kv_start));
    for (int qh = 0; qh < num_q_heads; ++qh) {
        const int kvh = qh / group;
        const float *qr = q + (size_t)qh * head_dim;
        double mx = -INFINITY;
        for (int p = kv_start; p < seq_len; ++p) {
            const float *kr = k + ((size_t)p * num_kv_heads + kvh) * head_dim;
            double dot = 0.0;
            for (int i = 0; i < head_dim; ++i) dot += (double)qr[i] * (double)kr[i];
            scores[(size_t)(p - kv_start)] = dot * sc;
            mx = std::max(mx, dot * sc);
        }
        double sum = 0.0;
        for (int p = kv_start; p < seq_len; ++p) {
            scores[(size_t)(p - kv_start)] = std::exp(scores[(size_t)(p - kv_start)] - mx);
            sum += scores[(size_t)(p - kv_start)];
        }
        for (int i = 0; i < head_dim; ++i) {
            double acc = 0.0;
            for (int p = kv_start; p < seq_len; ++p) acc += scores[(size_t)(p - kv_start)] * (double)v[((size_t)p * num_kv_heads + kvh) * head_dim + i];
            out[(size_t)qh * head_dim + i] = sum > 0.0 ? (float)(acc / sum) : 0.0f;
        }
    }
}

// Kernel-order restatement of the split-KV decode path (M/Attention/attention.metal:135-222 attention_decode_partial and
// :339-377 attention_decode_combine; K/Attention/Attention.swift:128-147 for the split): fp16 inputs, the online-softmax
// recurrence in fp32 position by position inside each of num_chunks chunks of chunk_len positions, the un-normalized
// partial (m, d, o) per chunk, then the merge and the fp16 result.  ring_capacity != 0: position p lives in row
// p % ring_capacity of k / v (attn_ring_slot, :76-81).  Physical k, v: [rows, num_kv_heads, head_dim] fp16.
void tfo_k_attention_split(const uint16_t *q_f16, const uint16_t *k_f16, const uint16_t *v_f16, int head_dim, int num_q_heads,
                           int num_kv_heads, int seq_len, int kv_start, int chunk_len, int num_chunks, float scale, int ring_capacity,
                           uint16_t *out_f16) {
    const int group = num_q_heads / num_kv_heads;
    std::vector<float> m((size_t)num_chunks), d((size_t)num_chunks), o((size_t)num_chunks * head_dim);
    for (int qh = 0; qh < num_q_heads; ++qh) {
        const int kvh = qh / group;
        for (int c = 0; c < num_chunks; ++c) {
            const int p_start = kv_start + c * chunk_len, p_end = std::min(p_start + chunk_len, seq_len);
            float m_run = -INFINITY, d_run = 0.0f;
            float *oc = o.data() + (size_t)c * head_dim;
            for (int i = 0; i < head_dim; ++i) oc[i] = 0.0f;
            for (int p = p_start; p < p_end; ++p) {
                const int row = ring_capacity ? p % ring_capacity : p;
                const uint16_t *kr = k_f16 + ((size_t)row * num_kv_heads + kvh) * head_dim;
                const uint16_t *vr = v_f16 + ((size_t)row * num_kv_heads + kvh) * head_dim;
                float s = 0.0f;
                for (int i = 0; i < head_dim; ++i) s = std::fma(tfo_f16_to_float(q_f16[(size_t)qh * head_dim + i]), tfo_f16_to_float(kr[i]), s);
                s *= scale;
                const float m_new = std::max(m_run, s);
                const float alpha = std::exp(m_run - m_new), p_exp = std::exp(s - m_new);
                d_run = d_run * alpha + p_exp;
                for (int i = 0; i < head_dim; ++i) oc[i] = oc[i] * alpha + p_exp * tfo_f16_to_float(vr[i]);
                m_run = m_new;
            }
            m[(size_t)c] = m_run;
            d[(size_t)c] = d_run;
        }
        float m_glob = -INFINITY;
        for (int c = 0; c < num_chunks; ++c) m_glob = std::max(m_glob, m[(size_t)c]);
        float D = 0.0f;
        for (int c = 0; c < num_chunks; ++c) D += d[(size_t)c] * std::exp(m[(size_t)c] - m_glob);
        const float inv_d = D > 0.0f ? 1.0f / D : 0.0f;
        for (int i = 0; i < head_dim; ++i) {
            float acc = 0.0f;
            for (int c = 0; c < num_chunks; ++c) acc += o[(size_t)c * head_dim + i] * std::exp(m[(size_t)c] - m_glob);
            out_f16[(size_t)qh * head_dim + i] = tfo_f16_bits(acc * inv_d);
        }
    }
}

// K/Attention/Attention.swift:122-147 (Attention.chunkCount / splitGeometry): out = {effectiveLength, numChunks, chunkLength,
// partialThreadgroups, useSWAGroupedPartial}
void tfo_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, uint32_t kv_start, int prefer_gqa_swa,
                                  int32_t *out5) {
    const int q_per_kv = (int)(num_q_heads / num_kv_heads);
    const bool grouped = prefer_gqa_swa && q_per_kv <= 2;
    const int effective = (int)seq_len - (int)kv_start;
    const int eff = std::max(1, effective);
    const int default_chunks = grouped ? 8 : 16;
    const int base = std::max(1, std::min(default_chunks, std::min(64, eff)));
    const int chunks = grouped ? std::max(base, std::min(64, base * q_per_kv)) : base;
    out5[0] = effective;
    out5[1] = chunks;
    out5[2] = (eff + chunks - 1) / chunks;
    out5[3] = (grouped ? (int)num_kv_heads : (int)num_q_heads) * chunks;
    out5[4] = grouped ? 1 : 0;
}

// ---------------------------------------------------------------------------------------------------- attention (prefill)
// T/Core/Kernels/Attention/PrefillAttentionTests.swift:310-352 (reference): query t of the block sits at position
// start + t and sees keys [first, last) with first = max(0, start + t + 1 - window) (window 0: none) and
// last = min(kv_valid, start + t + 1).  q [chunk, q_stride], k / v [rows, kv_stride], out compact [chunk, q_heads, head_dim].
// Accumulation in double.
void tfo_prefill_attention_ref(const float *q, const float *k, const float *v, int start, int chunk, int head_dim, int q_heads, int kv_heads,
                               int kv_valid, int window, int q_stride, int kv_stride, float scale, float *out) {
    const int q_per_kv = q_heads / kv_heads;
    std::vector<double> w;
    for (int t = 0; t < chunk; ++t) {
        const int abs_q = start + t;
        const int first = window == 0 ? 0 : std::max(0, abs_q + 1 - window);
        const int last = std::min(kv_valid, abs_q + 1);
        for (int qh = 0; qh < q_heads; ++qh) {
            const int kvh = qh / q_per_kv;
            w.assign((size_t)std::max(0, last - first), 0.0);
            double mx = -INFINITY;
            for (int key = first; key < last; ++key) {
                double sc = 0.0;
                for (int d = 0; d < head_dim; ++d)
                    sc += (double)q[(size_t)t * q_stride + (size_t)qh * head_dim + d] * (double)k[(size_t)key * kv_stride + (size_t)kvh * head_dim + d];
                w[(size_t)(key - first)] = sc * (double)scale;
                mx = std::max(mx, sc * (double)scale);
            }
            double denom = 0.0;
            for (double &x : w) {
                x = std::exp(x - mx);
                denom += x;
            }
            for (int d = 0; d < head_dim; ++d) {
                double acc = 0.0;
                for (int key = first; key < last; ++key) acc += w[(size_t)(key - first)] * (double)v[(size_t)key * kv_stride + (size_t)kvh * head_dim + d];
                out[((size_t)t * q_heads + qh) * head_dim + d] = denom > 0.0 ? (float)(acc / denom) : 0.0f;
            }
        }
    }
}

// Kernel-order restatement of attention_prefill_causal_tiled (M/Prefill/prefill.metal:835-902): fp16 operands, one online
// softmax per (query, head) in fp32, key by key, fp16 result into out [chunk, o_stride]; ring_capacity != 0: key p lives in
// row p % ring_capacity.  Elements of out between rows are left as they are.
void tfo_k_prefill_attention(const uint16_t *q_f16, const uint16_t *k_f16, const uint16_t *v_f16, uint16_t *out_f16, int start, int chunk,
                             int head_dim, int q_heads, int kv_heads, int kv_valid, int window, int q_stride, int kv_stride, int o_stride,
                             float scale, int ring_capacity) {
    const int q_per_kv = q_heads / kv_heads;
    std::vector<float> acc((size_t)head_dim);
    for (int t = 0; t < chunk; ++t) {
        const int abs_q = start + t;
        const int first = (window != 0 && abs_q + 1 > window) ? abs_q + 1 - window : 0;
        const int last = std::min(kv_valid, abs_q + 1);
        for (int qh = 0; qh < q_heads; ++qh) {
            const int kvh = qh / q_per_kv;
            const uint16_t *qr = q_f16 + (size_t)t * q_stride + (size_t)qh * head_dim;
            float row_max = -INFINITY, row_sum = 0.0f;
            std::fill(acc.begin(), acc.end(), 0.0f);
            for (int key = first; key < last; ++key) {
                const int row = ring_capacity ? key % ring_capacity : key;
                const uint16_t *kr = k_f16 + (size_t)row * kv_stride + (size_t)kvh * head_dim;
                const uint16_t *vr = v_f16 + (size_t)row * kv_stride + (size_t)kvh * head_dim;
                float sc = 0.0f;
                for (int d = 0; d < head_dim; ++d) sc += tfo_f16_to_float(qr[d]) * tfo_f16_to_float(kr[d]);
                sc *= scale;
                const float new_max = std::max(row_max, sc);
                const float old_scale = row_sum > 0.0f ? std::exp(row_max - new_max) : 0.0f;
                const float new_scale = std::exp(sc - new_max);
                for (int d = 0; d < head_dim; ++d) acc[(size_t)d] = std::fma(new_scale, tfo_f16_to_float(vr[d]), acc[(size_t)d] * old_scale);
                row_sum = row_sum * old_scale + new_scale;
                row_max = new_max;
            }
            uint16_t *orow = out_f16 + (size_t)t * o_stride + (size_t)qh * head_dim;
            for (int d = 0; d < head_dim; ++d) orow[d] = tfo_f16_bits(row_sum > 0.0f ? acc[(size_t)d] / row_sum : 0.0f);
        }
    }
}

// ---------------------------------------------------------------------------------------------------- RoPE, QKV epilogue
// V/Support/Reference/Attention/RoPE.swift:82-128 (RopeRef.applyNeox): pairs (x[i], x[i + head_dim / 2]) for
// i < rotated_pairs rotate by angle position * theta^(-2 i / head_dim); everything else passes through.  fp32 in / out;
// the angle and its cosine / sine in double (the reference uses vForce, whose rounding is not specified).
void tfo_rope_neox_ref(const float *input, int num_tokens, int num_heads, int head_dim, int rotated_pairs, int position, float theta,
                       float *out) {
    const int half_dim = head_dim / 2;
    for (size_t i = 0; i < (size_t)num_tokens * num_heads * head_dim; ++i) out[i] = input[i];
    for (int k = 0; k < rotated_pairs; ++k) {
        const double angle = (double)position * std::pow((double)theta, -(double)(2 * k) / (double)head_dim);
        const double c = std::cos(angle), sn = std::sin(angle);
        for (int th = 0; th < num_tokens * num_heads; ++th) {
            const size_t base = (size_t)th * head_dim;
            const double x0 = input[base + k], x1 = input[base + half_dim + k];
            out[base + k] = (float)(x0 * c - x1 * sn);
            out[base + half_dim + k] = (float)(x0 * sn + x1 * c);
        }
    }
}

// Kernel-order restatement of rope_default_neox / rope_proportional_neox (M/Primitives/rope.metal:33-96): fp16 data in
// place, fp32 arithmetic, fp16 results.
void tfo_k_rope_neox(uint16_t *data_f16, int num_tokens, int num_heads, int head_dim, int rotated_pairs, uint32_t position, float theta) {
    const int half_dim = head_dim / 2;
    for (int th = 0; th < num_tokens * num_heads; ++th) {
        uint16_t *head = data_f16 + (size_t)th * head_dim;
        for (int pair = 0; pair < rotated_pairs; ++pair) {
            const float exponent = -(float)(2u * (uint32_t)pair) / (float)head_dim;
            const float angle = (float)position * std::pow(theta, exponent);
            const float c = std::cos(angle), sn = std::sin(angle);
            const float x0 = tfo_f16_to_float(head[pair]), x1 = tfo_f16_to_float(head[half_dim + pair]);
            head[pair] = tfo_f16_bits(x0 * c - x1 * sn);
            head[half_dim + pair] = tfo_f16_bits(x0 * sn + x1 * c);
        }
    }
}

// Kernel-order restatement of fused_qkv_epilogue (M/Fusions/fused.metal:84-173): per head RMSNorm (q and k with their
// bf16 weight, v without), the normalized values rounded to fp16, then NeoX RoPE on the first rotated_pairs pairs of q
// and k; all in place.
void tfo_k_fused_qkv_epilogue(uint16_t *q_f16, uint16_t *k_f16, uint16_t *v_f16, const uint16_t *q_weight_bf16, const uint16_t *k_weight_bf16,
                              int head_dim, int num_q_heads, int num_kv_heads, uint32_t position, float theta, int rotated_pairs, float eps) {
    std::vector<uint16_t> normed((size_t)head_dim);
    for (int hg = 0; hg < num_q_heads + 2 * num_kv_heads; ++hg) {
        const bool is_q = hg < num_q_heads, is_k = !is_q && hg < num_q_heads + num_kv_heads;
        uint16_t *dst = is_q ? q_f16 + (size_t)hg * head_dim
                             : (is_k ? k_f16 + (size_t)(hg - num_q_heads) * head_dim : v_f16 + (size_t)(hg - num_q_heads - num_kv_heads) * head_dim);
        const uint16_t *w = is_q ? q_weight_bf16 : k_weight_bf16;
        const float inv = 1.0f / std::sqrt(k_block_sum_squares(dst, head_dim) / (float)head_dim + eps);
        for (int i = 0; i < head_dim; ++i) {
            float xv = tfo_f16_to_float(dst[i]) * inv;
            if (is_q || is_k) xv *= tfo_bf16_to_float(w[i]);
            normed[(size_t)i] = tfo_f16_bits(xv);
        }
        for (int i = 0; i < head_dim; ++i) dst[i] = normed[(size_t)i];
        if (is_q || is_k) tfo_k_rope_neox(dst, 1, 1, head_dim, rotated_pairs, position, theta);
    }
}

}  // extern "C"
