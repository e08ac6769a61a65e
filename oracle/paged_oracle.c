/*
 * CPU oracle for the paged-KV attention path -- TEST INFRASTRUCTURE ONLY.
 * See paged_oracle.h for what each function restates and how it is pinned.
 * Build: make -C oracle   (plain gcc, -O3, no -march, like the reference's
 * CMakeLists.txt:22-30; -fopenmp only parallelises the outer pair loop).
 */
#include "paged_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 */

float oracle_fp16_to_float(uint16_t h) {
    /* compiler/runtime/float_convert.hpp:14-48 */
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t sig = h & 0x03FFu;
    uint32_t word;
    if (e == 0) {
        if (sig == 0) {
            word = sign;
        } else {
            /* subnormal: normalise the significand */
            uint32_t shift = 0;
            while ((sig & 0x0400u) == 0) {
                sig <<= 1;
                ++shift;
            }
            sig &= 0x03FFu;
            word = sign | ((127u - 14u - shift) << 23) | (sig << 13);
        }
    } else if (e == 0x1Fu) {
        word = sign | (255u << 23) | (sig << 13);
    } else {
        word = sign | ((e - 15u + 127u) << 23) | (sig << 13);
    }
    float f;
    memcpy(&f, &word, sizeof f);
    return f;
}

uint16_t oracle_float_to_fp16_ref(float value) {
    /* compiler/runtime/float_convert.hpp:57-76 */
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t e = (int32_t)((bits >> 23) & 0xFFu) - 127 + 15;
    uint32_t man = bits & 0x7FFFFFu;
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man = (man | 0x800000u) >> (1 - e);
        return (uint16_t)(sign | ((man + 0x1000u) >> 13));
    }
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint32_t)e << 10) | ((man + 0x1000u) >> 13));
}

uint16_t oracle_float_to_fp16_rne(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    uint32_t sign = (bits >> 16) & 0x8000u;
    uint32_t absb = bits & 0x7FFFFFFFu;
    if (absb >= 0x7F800000u) { /* inf / nan */
        uint32_t man = absb & 0x7FFFFFu;
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7C00u | 0x0200u | (man >> 13));
    }
    if (absb >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absb < 0x38800000u) { /* below the smallest normal half, 2^-14 */
        if (absb < 0x33000000u) return (uint16_t)sign; /* < 2^-25 */
        int32_t e = (int32_t)(absb >> 23);             /* biased fp32 exponent */
        uint32_t man = (absb & 0x7FFFFFu) | 0x800000u;
        int shift = 126 - e; /* result = man >> shift in units of 2^-24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (absb >> 23) - 127u + 15u;
    uint32_t man = absb & 0x7FFFFFu;
    uint32_t q = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
}

void oracle_fp16_to_float_n(const uint16_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_fp16_to_float(src[i]);
}
void oracle_float_to_fp16_ref_n(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_float_to_fp16_ref(src[i]);
}
void oracle_float_to_fp16_rne_n(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_float_to_fp16_rne(src[i]);
}

/* ------------------------------------------------------- scatter / gather */

int oracle_scatter_kv_paged_batched_f16(uint16_t* page_storage,
                                        const uint32_t* page_ids,
                                        const uint32_t* slots_in_page,
                                        size_t page_size_tokens,
                                        size_t n_kv_heads,
                                        size_t head_dim,
                                        size_t batch,
                                        const uint16_t* src) {
    /* host checks: metal_runtime.mm:7241-7243 */
    if (!page_storage || !src || !page_ids || !slots_in_page) return 0;
    if (batch == 0 || n_kv_heads == 0 || head_dim == 0 || page_size_tokens == 0) return 0;
    const size_t elements_per_page = page_size_tokens * n_kv_heads * head_dim;
    /* kernel: metal_runtime.mm:413-423 */
    for (size_t req = 0; req < batch; ++req) {
        for (size_t kv = 0; kv < n_kv_heads; ++kv) {
            for (size_t dim = 0; dim < head_dim; ++dim) {
                size_t gid = (req * n_kv_heads + kv) * head_dim + dim;
                size_t dst = (size_t)page_ids[req] * elements_per_page +
                             (size_t)slots_in_page[req] * (n_kv_heads * head_dim) +
                             kv * head_dim + dim;
                page_storage[dst] = src[gid];
            }
        }
    }
    return 1;
}

int oracle_scatter_kv_paged(void* page_storage,
                            const uint32_t* page_table, size_t n_page_table,
                            size_t page_size_tokens, size_t n_kv_heads,
                            size_t head_dim, size_t tokens, size_t start_slot,
                            const void* src, size_t dtype_bytes) {
    /* host checks: metal_runtime.mm:7839-7845 */
    if (!page_storage || !src) return 0;
    if (page_size_tokens == 0 || n_kv_heads == 0 || head_dim == 0 || tokens == 0) return 0;
    if (dtype_bytes != 2 && dtype_bytes != 4) return 0;
    if (start_slot >= page_size_tokens) return 0;
    size_t needed = (start_slot + tokens + page_size_tokens - 1) / page_size_tokens;
    if (n_page_table < needed) return 0;
    const size_t epp = page_size_tokens * n_kv_heads * head_dim;
    /* kernel: metal_runtime.mm:474-489; src is [kv][token][dim] */
    for (size_t kv = 0; kv < n_kv_heads; ++kv) {
        for (size_t token = 0; token < tokens; ++token) {
            size_t absolute_slot = start_slot + token;
            size_t page_idx = absolute_slot / page_size_tokens;
            size_t slot = absolute_slot % page_size_tokens;
            size_t dst = (size_t)page_table[page_idx] * epp + slot * n_kv_heads * head_dim +
                         kv * head_dim;
            size_t s = (kv * tokens + token) * head_dim;
            memcpy((char*)page_storage + dst * dtype_bytes, (const char*)src + s * dtype_bytes,
                   head_dim * dtype_bytes);
        }
    }
    return 1;
}

int oracle_gather_kv_pages(const void* page_storage,
                           const uint32_t* page_table, size_t n_page_table,
                           size_t page_size_tokens, size_t n_kv_heads,
                           size_t head_dim, size_t num_tokens,
                           void* dst, size_t dtype_bytes) {
    /* host checks: metal_runtime.mm:7657-7662 */
    if (!page_storage || !dst) return 0;
    if (page_size_tokens == 0 || n_kv_heads == 0 || head_dim == 0 || num_tokens == 0) return 0;
    if (dtype_bytes != 2 && dtype_bytes != 4) return 0;
    size_t needed = (num_tokens + page_size_tokens - 1) / page_size_tokens;
    if (n_page_table < needed) return 0;
    const size_t epp = page_size_tokens * n_kv_heads * head_dim;
    /* kernel: metal_runtime.mm:334-347; dst is [head][token][dim] */
    for (size_t head = 0; head < n_kv_heads; ++head) {
        for (size_t tok = 0; tok < num_tokens; ++tok) {
            size_t page_idx = tok / page_size_tokens;
            size_t slot = tok % page_size_tokens;
            size_t s = (size_t)page_table[page_idx] * epp + slot * n_kv_heads * head_dim +
                       head * head_dim;
            size_t d = (head * num_tokens + tok) * head_dim;
            memcpy((char*)dst + d * dtype_bytes, (const char*)page_storage + s * dtype_bytes,
                   head_dim * dtype_bytes);
        }
    }
    return 1;
}

/* ------------------------------------------------- qkv split + RoPE + cast */

size_t oracle_rotary_coefficients(size_t position, size_t rotary_dim, float freq_base,
                                  float freq_scale, float* cos_out, float* sin_out) {
    /* quantization.cpp:801-822 */
    if (rotary_dim < 2) return 0;
    if (freq_base <= 0.0f) freq_base = 10000.0f;
    if (freq_scale == 0.0f) freq_scale = 1.0f;
    size_t pairs = rotary_dim / 2;
    float pos = (float)position;
    for (size_t i = 0; i < pairs; ++i) {
        float exponent = (float)(2 * i) / (float)rotary_dim;
        float inv_freq = powf(freq_base, -exponent);
        float angle = pos * inv_freq * freq_scale;
        cos_out[i] = cosf(angle);
        sin_out[i] = sinf(angle);
    }
    return pairs;
}

int oracle_qkv_split_rope_cast(const float* qkv, float* q, float* k, float* v,
                               uint16_t* k_f16, uint16_t* v_f16,
                               const float* cos_table, const float* sin_table,
                               size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                               size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                               size_t rotary_dim) {
    if (!qkv || !q || !k || !v || !k_f16 || !v_f16) return 0;
    if (batch == 0 || num_heads == 0 || kv_heads == 0 || head_dim == 0) return 0;
    if (q_rows + k_rows + v_rows > qkv_rows) return 0;
    if (q_rows != num_heads * head_dim || k_rows != kv_heads * head_dim) return 0;
    if (rotary_dim > head_dim || (rotary_dim & 1)) return 0;
    if (rotary_dim > 0 && (!cos_table || !sin_table)) return 0;
    /* split: metal_runtime.mm:447-455 with offsets 0, q_rows, q_rows + k_rows (:7962-7964) */
    for (size_t r = 0; r < batch; ++r) {
        memcpy(q + r * q_rows, qkv + r * qkv_rows, q_rows * sizeof(float));
        memcpy(k + r * k_rows, qkv + r * qkv_rows + q_rows, k_rows * sizeof(float));
        memcpy(v + r * v_rows, qkv + r * qkv_rows + q_rows + k_rows, v_rows * sizeof(float));
    }
    /* rope on q (num_heads) and k (kv_heads): metal_runtime.mm:287-314, :7989-7990 */
    const size_t pairs = rotary_dim / 2;
    for (int which = 0; which < 2 && pairs; ++which) {
        float* data = which ? k : q;
        const size_t nh = which ? kv_heads : num_heads;
        for (size_t r = 0; r < batch; ++r)
            for (size_t h = 0; h < nh; ++h)
                for (size_t p = 0; p < pairs; ++p) {
                    float* x = data + (r * nh + h) * head_dim + 2 * p;
                    const float c = cos_table[r * pairs + p], s = sin_table[r * pairs + p];
                    const float x0 = x[0], x1 = x[1];
                    const float a0 = x0 * c, a1 = x1 * s, b0 = x0 * s, b1 = x1 * c;
                    x[0] = a0 - a1;
                    x[1] = b0 + b1;
                }
    }
    /* casts: metal_runtime.mm:457-464, :8009-8010 */
    oracle_float_to_fp16_rne_n(k, k_f16, batch * k_rows);
    oracle_float_to_fp16_rne_n(v, v_f16, batch * v_rows);
    return 1;
}

/* ------------------------------------------------ walker layer operators */

int oracle_rms_norm_batched(const float* in, const float* weight, size_t n_weight, float epsilon,
                            size_t batch, size_t length, float* out) {
    if (!in || !out || batch == 0 || length == 0) return 0;
    for (size_t r = 0; r < batch; ++r) {
        const float* x = in + r * length;
        float mean_sq = 0.0f; /* operator_backend.cpp:194-198 */
        for (size_t i = 0; i < length; ++i) mean_sq += x[i] * x[i];
        mean_sq = mean_sq / (float)length;
        float inv = 1.0f / sqrtf(mean_sq + epsilon);
        for (size_t i = 0; i < length; ++i) {
            float gamma = (weight && i < n_weight) ? weight[i] : 1.0f;
            out[r * length + i] = x[i] * inv * gamma;
        }
    }
    return 1;
}

int oracle_add(const float* a, const float* b, float* out, size_t n) {
    if (!a || !b || !out || n == 0) return 0;
    for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
    return 1;
}

int oracle_silu_mul(const float* gate, const float* up, float* out, size_t n) {
    if (!gate || !up || !out || n == 0) return 0;
    for (size_t i = 0; i < n; ++i) {
        float g = gate[i];
        float silu = g / (1.0f + expf(-g));
        out[i] = silu * up[i];
    }
    return 1;
}

int oracle_gate_up_split_silu_mul(const float* gate_up, float* gate, float* up, float* out,
                                  size_t batch, size_t ffn_inner, size_t gate_up_rows) {
    if (!gate_up || !gate || !up || !out || batch == 0 || ffn_inner == 0) return 0;
    if (2 * ffn_inner > gate_up_rows) return 0;
    for (size_t r = 0; r < batch; ++r) {
        memcpy(gate + r * ffn_inner, gate_up + r * gate_up_rows, ffn_inner * sizeof(float));
        memcpy(up + r * ffn_inner, gate_up + r * gate_up_rows + ffn_inner, ffn_inner * sizeof(float));
    }
    return oracle_silu_mul(gate, up, out, batch * ffn_inner);
}

int oracle_matmul_q4_0_batched(const uint8_t* weights, const float* in, size_t batch, size_t rows,
                               size_t cols, size_t row_stride, float* out, int n_threads) {
    if (!weights || !in || !out || batch == 0 || rows == 0 || cols == 0) return 0;
    if (cols < 64 || (rows % 4u) != 0) return 0; /* metal_runtime.mm:6942 */
    const size_t nb = (cols + 31) / 32;
    if (row_stride < nb * 18) return 0;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(static)
    for (long long r = 0; r < (long long)rows; ++r) {
        const uint8_t* row = weights + (size_t)r * row_stride;
        for (size_t b = 0; b < batch; ++b) {
            const float* vec = in + b * cols;
            float acc = 0.0f; /* quantization.cpp:247-267 */
            for (size_t blk = 0; blk < nb; ++blk) {
                const size_t base = blk * 32;
                const uint8_t* p = row + blk * 18;
                uint16_t dh;
                memcpy(&dh, p, 2);
                const float d = oracle_fp16_to_float(dh);
                for (size_t j = 0; j < 16; ++j) {
                    const uint8_t byte = p[2 + j];
                    const int lo = (int)(byte & 0x0F) - 8;
                    const int hi = (int)((byte >> 4) & 0x0F) - 8;
                    if (base + j < cols) acc += d * (float)lo * vec[base + j];
                    if (base + j + 16 < cols) acc += d * (float)hi * vec[base + j + 16];
                }
            }
            out[b * rows + (size_t)r] = acc;
        }
    }
    return 1;
}

void oracle_quantize_row_q4_0(const float* src, size_t cols, uint8_t* dst) {
    const size_t blocks = (cols + 31) / 32;
    size_t idx = 0;
    for (size_t b = 0; b < blocks; ++b) {
        const float* block = src + idx;
        const size_t bs = cols - idx < 32 ? cols - idx : 32;
        float max_abs = 0.0f, max_val = 0.0f; /* quantization.cpp:283-292 */
        for (size_t i = 0; i < bs; ++i) {
            float v = block[i], av = fabsf(v);
            if (av > max_abs) {
                max_abs = av;
                max_val = v;
            }
        }
        const float scale = max_val / -8.0f;
        const float inv_scale = (scale != 0.0f) ? (1.0f / scale) : 0.0f;
        const uint16_t fp = oracle_float_to_fp16_ref(scale);
        uint8_t* o = dst + b * 18;
        memcpy(o, &fp, 2);
        for (size_t j = 0; j < 16; ++j) {
            const float x0 = (j < bs) ? block[j] * inv_scale : 0.0f;
            const float x1 = (j + 16 < bs) ? block[j + 16] * inv_scale : 0.0f;
            int q0 = (int)(x0 + 8.5f), q1 = (int)(x1 + 8.5f);
            q0 = q0 < 0 ? 0 : (q0 > 15 ? 15 : q0);
            q1 = q1 < 0 ? 0 : (q1 > 15 ? 15 : q1);
            o[2 + j] = (uint8_t)((q1 << 4) | q0);
        }
        idx += bs;
    }
}

/* ---- Q6_K (compiler/runtime/quantization.cpp:142-147: 256 weights per 210-byte block =
 * 128 bytes of low nibbles, 64 bytes of high bit pairs, 16 int8 group scales, fp16 d) */

/* dequantizeRowQ6_K, quantization.cpp:1469-1499, one block */
static void q6k_block_values(const uint8_t* block, float* y) {
    const uint8_t* ql = block;
    const uint8_t* qh = block + 128;
    const int8_t* sc = (const int8_t*)(block + 192);
    uint16_t dh;
    memcpy(&dh, block + 208, 2);
    const float d = oracle_fp16_to_float(dh);
    for (size_t n = 0; n < 256; n += 128) {
        for (int l = 0; l < 32; ++l) {
            const int is = l / 16;
            const int8_t q1 = (int8_t)((int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32);
            const int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            const int8_t q3 = (int8_t)((int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            const int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            y[l + 0] = d * (float)sc[is + 0] * (float)q1;
            y[l + 32] = d * (float)sc[is + 2] * (float)q2;
            y[l + 64] = d * (float)sc[is + 4] * (float)q3;
            y[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
        y += 128;
        ql += 64;
        qh += 32;
        sc += 8;
    }
}

void oracle_dequantize_row_q6_k(const uint8_t* src, size_t cols, float* dst) {
    const size_t nb = (cols + 255) / 256;
    for (size_t b = 0; b < nb; ++b) {
        float buf[256];
        q6k_block_values(src + b * 210, buf);
        const size_t n = cols - b * 256 < 256 ? cols - b * 256 : 256;
        memcpy(dst + b * 256, buf, n * sizeof(float));
    }
}

int oracle_matmul_q6_k_batched(const uint8_t* weights, const float* in, size_t batch, size_t rows,
                               size_t cols, size_t row_stride, float* out, int n_threads) {
    if (!weights || !in || !out || batch == 0 || rows == 0 || cols == 0) return 0;
    if (cols < 64 || (rows % 4u) != 0) return 0; /* metal_runtime.mm:6985 */
    const size_t nb = (cols + 255) / 256;
    if (row_stride < nb * 210) return 0;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(static)
    for (long long r = 0; r < (long long)rows; ++r) {
        const uint8_t* row = weights + (size_t)r * row_stride;
        float* tmp = (float*)malloc(nb * 256 * sizeof(float));
        for (size_t b = 0; b < nb; ++b) q6k_block_values(row + b * 210, tmp + b * 256);
        for (size_t b = 0; b < batch; ++b) {
            const float* vec = in + b * cols;
            float acc = 0.0f; /* dotProductRowQ6_K, quantization.cpp:1570-1586 */
            for (size_t i = 0; i < cols; ++i) acc += tmp[i] * vec[i];
            out[b * rows + (size_t)r] = acc;
        }
        free(tmp);
    }
    return 1;
}

static int q6k_clamp(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* quantizeRowQ6_K, quantization.cpp:1588-1663 */
void oracle_quantize_row_q6_k(const float* src, size_t cols, uint8_t* dst) {
    const size_t blocks = (cols + 255) / 256;
    size_t offset = 0;
    for (size_t b = 0; b < blocks; ++b) {
        const size_t be = cols - offset < 256 ? cols - offset : 256;
        float data[256] = {0};
        memcpy(data, src + offset, be * sizeof(float));
        float chunk_scale[16];
        float max_scale = 0.0f;
        for (size_t j = 0; j < 16; ++j) {
            const size_t start = j * 16;
            if (start >= be) {
                chunk_scale[j] = 0.0f;
                continue;
            }
            float max_abs = 0.0f;
            for (size_t i = start; i < start + 16 && i < be; ++i) max_abs = fmaxf(max_abs, fabsf(data[i]));
            float scale = max_abs / 32.0f;
            if (scale < 1e-8f) scale = 0.0f;
            chunk_scale[j] = scale;
            max_scale = fmaxf(max_scale, scale);
        }
        const float base = max_scale > 0.0f ? max_scale / 127.0f : 0.0f;
        uint8_t* out = dst + b * 210;
        const uint16_t dh = oracle_float_to_fp16_ref(base);
        memcpy(out + 208, &dh, 2);
        uint8_t enc[256];
        for (size_t j = 0; j < 16; ++j) {
            int8_t sc = 0;
            if (base > 0.0f && chunk_scale[j] > 0.0f)
                sc = (int8_t)q6k_clamp((int)roundf(chunk_scale[j] / base), -127, 127);
            out[192 + j] = (uint8_t)sc;
            const float actual = base * (float)sc;
            for (size_t i = 0; i < 16; ++i) {
                const size_t idx = j * 16 + i;
                const float value = idx < be ? data[idx] : 0.0f;
                const float qf = actual != 0.0f ? roundf(value / actual) : 0.0f;
                enc[idx] = (uint8_t)(q6k_clamp((int)qf, -32, 31) + 32);
            }
        }
        memset(out, 0, 192);
        uint8_t* ql = out;
        uint8_t* qh = out + 128;
        for (size_t n = 0; n < 256; n += 128) {
            for (size_t l = 0; l < 32; ++l) {
                const uint8_t q1 = enc[n + l], q2 = enc[n + l + 32], q3 = enc[n + l + 64], q4 = enc[n + l + 96];
                ql[l + 0] = (uint8_t)((q1 & 0xF) | ((q3 & 0xF) << 4));
                ql[l + 32] = (uint8_t)((q2 & 0xF) | ((q4 & 0xF) << 4));
                qh[l] = (uint8_t)(((q1 >> 4) & 3) | (((q2 >> 4) & 3) << 2) | (((q3 >> 4) & 3) << 4) |
                                  (((q4 >> 4) & 3) << 6));
            }
            ql += 64;
            qh += 32;
        }
        offset += be;
    }
}

/* ------------------------------------------------------------- attention */

static int attention_args_ok(const void* q, const void* k, const void* v, const void* o,
                             const uint32_t* flat, size_t n_flat, const uint32_t* off,
                             const uint32_t* seq, const uint32_t* qpos, size_t batch,
                             size_t num_heads, size_t kv_heads, size_t head_dim,
                             size_t page_size_tokens) {
    /* metal_runtime.mm:7742-7750 */
    if (!q || !k || !v || !o) return 0;
    if (batch == 0 || num_heads == 0 || head_dim == 0 || page_size_tokens == 0) return 0;
    if (kv_heads == 0 || (num_heads % kv_heads) != 0) return 0;
    if (!off || !seq || !qpos) return 0;
    if (n_flat < off[batch]) return 0;
    if (n_flat > 0 && !flat) return 0;
    if (head_dim > 256) return 0;
    return 1;
}

static inline size_t kv_row_offset(const uint32_t* flat, uint32_t pt_base, size_t pos,
                                   size_t page_size_tokens, size_t kv_heads, size_t head_dim,
                                   size_t kv_h) {
    /* metal_runtime.mm:2268-2273 */
    size_t page_idx = pos / page_size_tokens;
    size_t slot = pos - page_idx * page_size_tokens;
    size_t page_id = flat[pt_base + page_idx];
    return page_id * (page_size_tokens * kv_heads * head_dim) + slot * (kv_heads * head_dim) +
           kv_h * head_dim;
}

/* attention_cpu.cpp:99-105 */
static float dot_scalar(const float* lhs, const float* rhs, size_t dim) {
    float acc = 0.0f;
    for (size_t i = 0; i < dim; ++i) acc += lhs[i] * rhs[i];
    return acc;
}

/* One (request, head) pair in the executor-CPU order.  `limit` is the number
 * of visible kv positions (already reduced by the causal rule). */
static void executor_one_head(const float* q_head, const uint16_t* k_pages,
                              const uint16_t* v_pages, float* out_head,
                              const uint32_t* flat, uint32_t pt_base, size_t limit,
                              size_t kv_h, size_t kv_heads, size_t head_dim,
                              size_t page_size_tokens, float* logits, float* row) {
    const float inv_sqrt = 1.0f / sqrtf((float)head_dim); /* attention_cpu.cpp:441 */
    for (size_t d = 0; d < head_dim; ++d) out_head[d] = 0.0f;
    if (limit == 0) return; /* metal_runtime.mm:2254-2257 */
    for (size_t t = 0; t < limit; ++t) {
        /* readRow -> dequantizeRowTo (attention_cpu.cpp:191-201, 447) */
        size_t off = kv_row_offset(flat, pt_base, t, page_size_tokens, kv_heads, head_dim, kv_h);
        for (size_t d = 0; d < head_dim; ++d) row[d] = oracle_fp16_to_float(k_pages[off + d]);
        logits[t] = dot_scalar(q_head, row, head_dim) * inv_sqrt; /* :448 */
    }
    /* softmax, attention_cpu.cpp:21-33 */
    float max_val = logits[0];
    for (size_t t = 1; t < limit; ++t)
        if (logits[t] > max_val) max_val = logits[t];
    float sum = 0.0f;
    for (size_t t = 0; t < limit; ++t) {
        logits[t] = expf(logits[t] - max_val);
        sum += logits[t];
    }
    if (sum <= 0.0f) sum = 1.0f;
    for (size_t t = 0; t < limit; ++t) logits[t] /= sum;
    /* V axpy, attention_cpu.cpp:460-467 with accumulateScaled :166-170 */
    for (size_t t = 0; t < limit; ++t) {
        size_t off = kv_row_offset(flat, pt_base, t, page_size_tokens, kv_heads, head_dim, kv_h);
        for (size_t d = 0; d < head_dim; ++d) row[d] = oracle_fp16_to_float(v_pages[off + d]);
        float w = logits[t];
        for (size_t d = 0; d < head_dim; ++d) out_head[d] += w * row[d];
    }
}

static size_t visible_limit(uint32_t S, uint32_t q_pos, int apply_causal) {
    /* metal_runtime.mm:2286: kv_pos > q_pos is masked when causal */
    size_t limit = S;
    if (apply_causal && (size_t)q_pos + 1 < limit) limit = (size_t)q_pos + 1;
    return limit;
}

int oracle_paged_attention_executor(const float* q,
                                    const uint16_t* k_pages,
                                    const uint16_t* v_pages,
                                    float* out,
                                    const uint32_t* page_tables_flat, size_t n_flat,
                                    const uint32_t* page_table_offsets,
                                    const uint32_t* seq_lens,
                                    const uint32_t* q_positions,
                                    size_t batch, size_t num_heads, size_t kv_heads,
                                    size_t head_dim, size_t page_size_tokens,
                                    int apply_causal, int n_threads) {
    if (!attention_args_ok(q, k_pages, v_pages, out, page_tables_flat, n_flat,
                           page_table_offsets, seq_lens, q_positions, batch, num_heads,
                           kv_heads, head_dim, page_size_tokens))
        return 0;
    size_t max_s = 1;
    for (size_t r = 0; r < batch; ++r)
        if (seq_lens[r] > max_s) max_s = seq_lens[r];
    const long pairs = (long)(batch * num_heads);
    if (n_threads < 1) n_threads = 1;
#ifdef _OPENMP
#pragma omp parallel num_threads(n_threads)
#endif
    {
        float* logits = (float*)malloc(max_s * sizeof(float));
        float* row = (float*)malloc(head_dim * sizeof(float));
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (long p = 0; p < pairs; ++p) {
            size_t r = (size_t)p / num_heads;
            size_t h = (size_t)p % num_heads;
            size_t kv_h = h * kv_heads / num_heads; /* attention_cpu.cpp:443 */
            if (kv_h > kv_heads - 1) kv_h = kv_heads - 1;
            size_t limit = visible_limit(seq_lens[r], q_positions[r], apply_causal);
            executor_one_head(q + (r * num_heads + h) * head_dim, k_pages, v_pages,
                              out + (r * num_heads + h) * head_dim, page_tables_flat,
                              page_table_offsets[r], limit, kv_h, kv_heads, head_dim,
                              page_size_tokens, logits, row);
        }
        free(logits);
        free(row);
    }
    return 1;
}

int oracle_paged_attention_flashref(const float* q,
                                    const uint16_t* k_pages,
                                    const uint16_t* v_pages,
                                    float* out,
                                    const uint32_t* page_tables_flat, size_t n_flat,
                                    const uint32_t* page_table_offsets,
                                    const uint32_t* seq_lens,
                                    const uint32_t* q_positions,
                                    size_t batch, size_t num_heads, size_t kv_heads,
                                    size_t head_dim, size_t page_size_tokens,
                                    int apply_causal) {
    if (!attention_args_ok(q, k_pages, v_pages, out, page_tables_flat, n_flat,
                           page_table_offsets, seq_lens, q_positions, batch, num_heads,
                           kv_heads, head_dim, page_size_tokens))
        return 0;
    /* tests/test_paged_flash.cpp:32-90 */
    const float inv_sqrt_d = 1.0f / sqrtf((float)head_dim);
    size_t max_s = 1;
    for (size_t r = 0; r < batch; ++r)
        if (seq_lens[r] > max_s) max_s = seq_lens[r];
    float* scores = (float*)malloc(max_s * sizeof(float));
    float* ws = (float*)malloc(max_s * sizeof(float));
    for (size_t r = 0; r < batch; ++r) {
        const size_t S = seq_lens[r];
        const size_t qpos = q_positions[r];
        const uint32_t base = page_table_offsets[r];
        for (size_t h = 0; h < num_heads; ++h) {
            size_t kv_h = (h * kv_heads) / num_heads;
            const float* qh = q + (r * num_heads + h) * head_dim;
            float* oh = out + (r * num_heads + h) * head_dim;
            float max_score = -INFINITY;
            for (size_t pos = 0; pos < S; ++pos) {
                size_t off = kv_row_offset(page_tables_flat, base, pos, page_size_tokens,
                                           kv_heads, head_dim, kv_h);
                float dot = 0.0f;
                for (size_t d = 0; d < head_dim; ++d)
                    dot += qh[d] * oracle_fp16_to_float(k_pages[off + d]);
                float scaled = dot * inv_sqrt_d;
                if (apply_causal && pos > qpos) scaled = -INFINITY;
                scores[pos] = scaled;
                if (scaled > max_score) max_score = scaled;
            }
            float sum = 0.0f;
            for (size_t pos = 0; pos < S; ++pos) {
                float e = (scores[pos] == -INFINITY) ? 0.0f : expf(scores[pos] - max_score);
                ws[pos] = e;
                sum += e;
            }
            float inv_sum = (sum > 0.0f) ? (1.0f / sum) : 0.0f;
            for (size_t d = 0; d < head_dim; ++d) {
                float acc = 0.0f;
                for (size_t pos = 0; pos < S; ++pos) {
                    size_t off = kv_row_offset(page_tables_flat, base, pos, page_size_tokens,
                                               kv_heads, head_dim, kv_h);
                    acc += ws[pos] * oracle_fp16_to_float(v_pages[off + d]);
                }
                oh[d] = acc * inv_sum;
            }
        }
    }
    free(scores);
    free(ws);
    return 1;
}

int oracle_paged_attention_prefill(const uint16_t* q_f16,
                                   const uint16_t* k_pages,
                                   const uint16_t* v_pages,
                                   float* out,
                                   const uint32_t* page_tables_flat, size_t n_flat,
                                   const uint32_t* page_table_offsets,
                                   const uint32_t* seq_lens,
                                   const uint32_t* q_start,
                                   size_t batch, size_t chunk, size_t num_heads,
                                   size_t kv_heads, size_t head_dim,
                                   size_t page_size_tokens, int n_threads) {
    if (!q_f16 || !k_pages || !v_pages || !out || !page_table_offsets || !seq_lens || !q_start)
        return 0;
    if (batch == 0 || chunk == 0 || num_heads == 0 || head_dim == 0 || page_size_tokens == 0)
        return 0;
    if (kv_heads == 0 || (num_heads % kv_heads) != 0 || head_dim > 256) return 0;
    if (n_flat < page_table_offsets[batch]) return 0;
    size_t max_s = 1;
    for (size_t r = 0; r < batch; ++r)
        if (seq_lens[r] > max_s) max_s = seq_lens[r];
    const long rows = (long)(batch * chunk * num_heads);
    if (n_threads < 1) n_threads = 1;
#ifdef _OPENMP
#pragma omp parallel num_threads(n_threads)
#endif
    {
        float* logits = (float*)malloc(max_s * sizeof(float));
        float* row = (float*)malloc(head_dim * sizeof(float));
        float* qf = (float*)malloc(head_dim * sizeof(float));
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 4)
#endif
        for (long p = 0; p < rows; ++p) {
            size_t h = (size_t)p % num_heads;
            size_t i = ((size_t)p / num_heads) % chunk;
            size_t r = (size_t)p / (num_heads * chunk);
            size_t kv_h = h * kv_heads / num_heads;
            const uint16_t* qrow = q_f16 + (size_t)p * head_dim;
            for (size_t d = 0; d < head_dim; ++d) qf[d] = oracle_fp16_to_float(qrow[d]);
            size_t limit = visible_limit(seq_lens[r], q_start[r] + (uint32_t)i, 1);
            executor_one_head(qf, k_pages, v_pages, out + (size_t)p * head_dim,
                              page_tables_flat, page_table_offsets[r], limit, kv_h, kv_heads,
                              head_dim, page_size_tokens, logits, row);
        }
        free(logits);
        free(row);
        free(qf);
    }
    return 1;
}

/* --------------------------------------------------------------- metrics */

void oracle_metrics(const float* a, const float* b, size_t n,
                    double* max_abs, double* mean_abs, double* rms, double* cosine) {
    /* parity_harness.cpp:233-255 */
    double mx = 0.0, sa = 0.0, sq = 0.0, dot = 0.0, na2 = 0.0, nb2 = 0.0;
    for (size_t i = 0; i < n; ++i) {
        double av = a[i], bv = b[i];
        double d = av - bv;
        double ad = fabs(d);
        if (ad > mx) mx = ad;
        sa += ad;
        sq += d * d;
        dot += av * bv;
        na2 += av * av;
        nb2 += bv * bv;
    }
    if (max_abs) *max_abs = mx;
    if (mean_abs) *mean_abs = n ? sa / (double)n : 0.0;
    if (rms) *rms = n ? sqrt(sq / (double)n) : 0.0;
    if (cosine) *cosine = (na2 > 0.0 && nb2 > 0.0) ? dot / (sqrt(na2) * sqrt(nb2)) : NAN;
}

double oracle_cosine(const float* a, const float* b, size_t n) {
    /* tests/test_paged_flash.cpp:93-102 */
    double dot = 0, na = 0, nb = 0;
    for (size_t i = 0; i < n; ++i) {
        dot += (double)a[i] * b[i];
        na += (double)a[i] * a[i];
        nb += (double)b[i] * b[i];
    }
    if (na == 0.0 || nb == 0.0) return 0.0;
    return dot / (sqrt(na) * sqrt(nb));
}

/* -------------------------------------------------------------- allocator */

struct oracle_page_pool {
    uint32_t capacity;
    uint32_t* free_list; /* LIFO: top of stack at free_list[n_free-1] */
    size_t n_free;
    size_t in_use;
};

oracle_page_pool* oracle_pool_new(uint32_t capacity) {
    /* paged_kv.cpp:10-17: id 0 at the top so a fresh pool counts upwards */
    oracle_page_pool* p = (oracle_page_pool*)malloc(sizeof *p);
    if (!p) return NULL;
    p->capacity = capacity;
    p->free_list = (uint32_t*)malloc((capacity ? capacity : 1) * sizeof(uint32_t));
    p->n_free = 0;
    p->in_use = 0;
    for (uint32_t i = capacity; i-- > 0;) p->free_list[p->n_free++] = i;
    return p;
}

void oracle_pool_free(oracle_page_pool* pool) {
    if (!pool) return;
    free(pool->free_list);
    free(pool);
}

int oracle_pool_allocate(oracle_page_pool* pool, uint32_t* id_out) {
    /* paged_kv.cpp:19-25 */
    if (pool->n_free == 0) return 0;
    *id_out = pool->free_list[--pool->n_free];
    ++pool->in_use;
    return 1;
}

int oracle_pool_allocate_n(oracle_page_pool* pool, size_t n, uint32_t* out) {
    /* paged_kv.cpp:27-35 */
    if (n > pool->n_free) return 0;
    for (size_t i = 0; i < n; ++i) out[i] = pool->free_list[--pool->n_free];
    pool->in_use += n;
    return 1;
}

void oracle_pool_release(oracle_page_pool* pool, uint32_t page_id) {
    /* paged_kv.cpp:37-42 */
    pool->free_list[pool->n_free++] = page_id;
    --pool->in_use;
}

size_t oracle_pool_in_use(const oracle_page_pool* pool) { return pool->in_use; }
size_t oracle_pool_free_count(const oracle_page_pool* pool) { return pool->n_free; }

size_t oracle_req_total_tokens(const oracle_request_kv* st) {
    /* paged_kv.hpp:73-77 */
    if (st->n_pages == 0) return 0;
    return (st->n_pages - 1) * (size_t)st->page_size_tokens + (size_t)st->tokens_in_last_page;
}

int oracle_req_reserve(oracle_request_kv* st, oracle_page_pool* pool, size_t target_tokens) {
    /* paged_kv.cpp:44-50; tokens_in_last_page is left alone, as there */
    if (st->page_size_tokens == 0) return 0;
    size_t needed = (target_tokens + st->page_size_tokens - 1) / st->page_size_tokens;
    if (needed <= st->n_pages) return 1;
    size_t to_alloc = needed - st->n_pages;
    if (st->n_pages + to_alloc > st->page_table_cap) return 0;
    if (!oracle_pool_allocate_n(pool, to_alloc, st->page_table + st->n_pages)) return 0;
    st->n_pages += to_alloc;
    return 1;
}

int oracle_req_extend_one_token(oracle_request_kv* st, oracle_page_pool* pool,
                                uint32_t* page_id, uint32_t* slot) {
    /* paged_kv.cpp:52-66 */
    if (st->page_size_tokens == 0) return 0;
    if (st->n_pages == 0 || st->tokens_in_last_page == st->page_size_tokens) {
        uint32_t id;
        if (st->n_pages >= st->page_table_cap) return 0;
        if (!oracle_pool_allocate(pool, &id)) return 0;
        st->page_table[st->n_pages++] = id;
        st->tokens_in_last_page = 0;
    }
    *page_id = st->page_table[st->n_pages - 1];
    *slot = st->tokens_in_last_page;
    ++st->tokens_in_last_page;
    return 1;
}

int oracle_req_locate(const oracle_request_kv* st, size_t pos, uint32_t* page_id,
                      uint32_t* slot) {
    /* paged_kv.cpp:68-75 */
    if (st->page_size_tokens == 0) return 0;
    if (pos >= oracle_req_total_tokens(st)) return 0;
    *page_id = st->page_table[pos / st->page_size_tokens];
    *slot = (uint32_t)(pos % st->page_size_tokens);
    return 1;
}

void oracle_req_release_all(oracle_request_kv* st, oracle_page_pool* pool) {
    /* paged_kv.cpp:77-81 */
    for (size_t i = 0; i < st->n_pages; ++i) oracle_pool_release(pool, st->page_table[i]);
    st->n_pages = 0;
    st->tokens_in_last_page = 0;
}
