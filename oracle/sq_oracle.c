/* CPU oracle for the codebook linear layer, scalar C.  TEST INFRASTRUCTURE ONLY.
 *
 * A second, independent restatement (beside oracle/sq_oracle.py) of the reference's CPU
 * arithmetic, used by the tests to cross-check the numpy oracle and to check the HIP
 * kernels at sizes where Python loops are too slow.  The shipped library never links it.
 *
 *   sqo_unpack   shapequant/packed.py:80-90     little-endian bit stream -> tags
 *   sqo_decode   shapequant/packed.py:259-270   w[r, perm[mask[r]][c]] = f32(table[...]) * f32(scale[r])
 *   sqo_linear   shapequant/kernels/gemv.py:3   y = x . W^T, double accumulation
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -shared -fPIC)
 */
#include <stdint.h>
#include <string.h>

/* IEEE binary16 -> binary32, exact. */
static float h2f(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u, u;
    if (e == 0) {
        if (m == 0) { u = s; }
        else {
            int k = 0;
            while (!(m & 1024u)) { m <<= 1; ++k; }
            u = s | (uint32_t)(113 - k) << 23 | (m & 1023u) << 13;
        }
    } else if (e == 31) { u = s | 0x7F800000u | m << 13; }
    else { u = s | (e + 112u) << 23 | m << 13; }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t tag_at(const int32_t* row, int64_t W, int bits, int64_t j) {
    int64_t p = j * bits, w = p >> 5;
    int s = (int)(p & 31);
    uint64_t lo = (uint32_t)row[w];
    uint64_t hi = (w + 1 < W) ? (uint32_t)row[w + 1] : 0u;
    return (uint32_t)(((lo | hi << 32) >> s) & ((1ull << bits) - 1ull));
}

void sqo_unpack(const int32_t* words, int64_t R, int64_t W, int bits, int64_t n, int64_t* out) {
    for (int64_t r = 0; r < R; ++r)
        for (int64_t j = 0; j < n; ++j)
            out[r * n + j] = tag_at(words + r * W, W, bits, j);
}

/* table: fp16 bits [G*K, d]; row_book / row_mask / perms may be NULL (perms int64 [M, C]). */
void sqo_decode(const int32_t* words, int64_t R, int64_t W, int bits, int64_t C, int d, int64_t K,
                const uint16_t* table, const uint16_t* row_scale, const uint8_t* row_book,
                const uint8_t* row_mask, const int64_t* perms, float* out) {
    int64_t nch = C / d;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        float s = h2f(row_scale[r]);
        int64_t base = row_book ? (int64_t)row_book[r] * K : 0;
        const int64_t* pm = (perms && row_mask) ? perms + (int64_t)row_mask[r] * C : 0;
        for (int64_t j = 0; j < nch; ++j) {
            const uint16_t* cw = table + (base + tag_at(words + r * W, W, bits, j)) * d;
            for (int k = 0; k < d; ++k) {
                int64_t c = j * d + k;
                out[r * C + (pm ? pm[c] : c)] = h2f(cw[k]) * s;
            }
        }
    }
}

/* y[b, r] = sum_c x[b, c] * w[r, c] in double. */
void sqo_linear(const float* x, int64_t B, const float* w, int64_t R, int64_t C, double* y) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r)
        for (int64_t b = 0; b < B; ++b) {
            double a = 0.0;
            for (int64_t c = 0; c < C; ++c) a += (double)x[b * C + c] * (double)w[r * C + c];
            y[b * R + r] = a;
        }
}
