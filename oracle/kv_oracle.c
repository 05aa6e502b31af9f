/*
 * Scalar C restatement of the data path of the KV-cache hot path.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libkv_oracle.so and loaded by
 * the tests and by the bench's CPU-baseline leg; the shipped library never
 * links or loads it.
 *
 * Each function restates, as plain loops, what the reference computes (paths
 * relative to the reference's deserve_worker/ package):
 *   orc_append        model/layer/attention.py:174-183 (append call site; the
 *                     kernel itself is in the absent flashinfer wheel)
 *   orc_gather        kvcache/manager.py:37-42  (pages[:, table] -> chunk)
 *   orc_scatter       kvcache/manager.py:63-73  (chunk -> pages[:, ids])
 *   orc_decode_attn   model/layer/attention.py:75-84,241-266 on the paged
 *                     layout consumed at attention.py:185
 *   orc_prefill_attn  same with the end-aligned causal mask (attention.py:188-192)
 *
 * Storage layout of one layer: (num_pages, 2, P, Hkv, D), K half then V half.
 * elt: 0 = fp32, 1 = fp16, 2 = bf16.  Attention accumulates in fp32 and writes
 * fp32.  These loops are deliberately independent of the numpy oracle (no
 * shared code) so the two cross-check each other.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline float load_elt(const void *base, int64_t idx, int elt)
{
    if (elt == 0) return ((const float *)base)[idx];
    uint16_t h = ((const uint16_t *)base)[idx];
    if (elt == 1) return half_to_float(h);
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline int elt_bytes(int elt) { return elt == 0 ? 4 : 2; }

static inline int64_t kv_len_of(const int32_t *kv_indptr, const int32_t *last, int b, int P)
{
    int64_t np = kv_indptr[b + 1] - kv_indptr[b];
    return np > 0 ? (np - 1) * P + last[b] : 0;
}

void orc_append(void *pages_layer, const void *k, const void *v, const int32_t *indptr,
                const int32_t *kv_indices, const int32_t *kv_indptr, const int32_t *last,
                int batch, int P, int Hkv, int D, int elt)
{
    const int64_t row = (int64_t)Hkv * D * elt_bytes(elt);
    const int64_t half = (int64_t)P * row;
    for (int b = 0; b < batch; b++) {
        int n = indptr[b + 1] - indptr[b];
        int64_t first = kv_len_of(kv_indptr, last, b, P) - n;
        for (int i = 0; i < n; i++) {
            int64_t pos = first + i;
            int64_t page = kv_indices[kv_indptr[b] + pos / P];
            int64_t slot = pos % P;
            char *dst = (char *)pages_layer + page * 2 * half + slot * row;
            memcpy(dst, (const char *)k + (int64_t)(indptr[b] + i) * row, row);
            memcpy(dst + half, (const char *)v + (int64_t)(indptr[b] + i) * row, row);
        }
    }
}

void orc_gather(void *chunk, const void *pool, const int32_t *ids, int n, int L,
                int64_t layer_stride_bytes, int64_t page_bytes)
{
    for (int l = 0; l < L; l++)
        for (int j = 0; j < n; j++)
            memcpy((char *)chunk + ((int64_t)l * n + j) * page_bytes,
                   (const char *)pool + l * layer_stride_bytes + (int64_t)ids[j] * page_bytes,
                   page_bytes);
}

void orc_scatter(void *pool, const void *chunk, const int32_t *ids, int n, int L,
                 int64_t layer_stride_bytes, int64_t page_bytes)
{
    for (int l = 0; l < L; l++)
        for (int j = 0; j < n; j++)
            memcpy((char *)pool + l * layer_stride_bytes + (int64_t)ids[j] * page_bytes,
                   (const char *)chunk + ((int64_t)l * n + j) * page_bytes,
                   page_bytes);
}

/* one (request, q head, query position) row of attention over kv [0, limit) */
static void attend_row(float *out, const void *q, int64_t q_off, const void *pages,
                       const int32_t *ids, int64_t limit, int kvh, int P, int Hkv, int D,
                       int elt, float scale, float *scores)
{
    const int64_t half = (int64_t)P * Hkv * D;
    float mx = -INFINITY;
    for (int64_t t = 0; t < limit; t++) {
        int64_t base = (int64_t)ids[t / P] * 2 * half + ((t % P) * Hkv + kvh) * (int64_t)D;
        float acc = 0.f;
        for (int d = 0; d < D; d++)
            acc += load_elt(q, q_off + d, elt) * load_elt(pages, base + d, elt);
        scores[t] = acc * scale;
        if (scores[t] > mx) mx = scores[t];
    }
    float sum = 0.f;
    for (int64_t t = 0; t < limit; t++) {
        scores[t] = expf(scores[t] - mx);
        sum += scores[t];
    }
    for (int d = 0; d < D; d++) out[d] = 0.f;
    for (int64_t t = 0; t < limit; t++) {
        int64_t base = (int64_t)ids[t / P] * 2 * half + half + ((t % P) * Hkv + kvh) * (int64_t)D;
        float p = scores[t] / sum;
        for (int d = 0; d < D; d++) out[d] += p * load_elt(pages, base + d, elt);
    }
}

void orc_decode_attn(float *out, const void *q, const void *pages_layer,
                     const int32_t *kv_indices, const int32_t *kv_indptr, const int32_t *last,
                     int batch, int Hq, int Hkv, int D, int P, int elt, float scale)
{
    const int rep = Hq / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < batch; b++) {
        for (int h = 0; h < Hq; h++) {
            int64_t T = kv_len_of(kv_indptr, last, b, P);
            float *scores = (float *)malloc(sizeof(float) * (size_t)(T > 0 ? T : 1));
            attend_row(out + ((int64_t)b * Hq + h) * D, q, ((int64_t)b * Hq + h) * D,
                       pages_layer, kv_indices + kv_indptr[b], T, h / rep, P, Hkv, D, elt,
                       scale, scores);
            free(scores);
        }
    }
}

void orc_prefill_attn(float *out, const void *q, const int32_t *qo_indptr, const void *pages_layer,
                      const int32_t *kv_indices, const int32_t *kv_indptr, const int32_t *last,
                      int batch, int Hq, int Hkv, int D, int P, int elt, float scale, int causal)
{
    const int rep = Hq / Hkv;
    for (int b = 0; b < batch; b++) {
        int n = qo_indptr[b + 1] - qo_indptr[b];
        int64_t T = kv_len_of(kv_indptr, last, b, P);
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
        for (int i = 0; i < n; i++) {
            for (int h = 0; h < Hq; h++) {
                int64_t limit = causal ? T - n + i + 1 : T;
                if (limit < 0) limit = 0;
                float *scores = (float *)malloc(sizeof(float) * (size_t)(T > 0 ? T : 1));
                int64_t row = ((int64_t)(qo_indptr[b] + i) * Hq + h) * D;
                attend_row(out + row, q, row, pages_layer, kv_indices + kv_indptr[b], limit,
                           h / rep, P, Hkv, D, elt, scale, scores);
                free(scores);
            }
        }
    }
}
