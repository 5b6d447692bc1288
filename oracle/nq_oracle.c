/* CPU oracle, C restatement.  TEST INFRASTRUCTURE ONLY: loaded by tests/ (and nothing in the
 * product) as an independent second opinion on oracle/nq_oracle.py.
 *
 * Follows, in the reference checkout:
 *   nqo_bit_position / nqo_pack_rows / nqo_unpack_rows
 *       src/nanoquant/kernel/utils.py:51-183   (bit = 1 encodes -1, column padding is +1)
 *   nqo_layer_forward_packed
 *       src/nanoquant/modules/linear.py:248-257 evaluated straight from the packed words in
 *       double precision: h = s_mid * sum_n sgn * (s_in*x), y = s_out * sum_r sgn * h
 *
 * Plain scalar loops on purpose: no shared code with the numpy oracle or the HIP kernels.
 */
#include <stdint.h>
#include <stdlib.h>

int nqo_bit_position(int k, int half2) {
    if (k < 0 || k > 31) return -1;
    if (!half2) return k;
    return 15 - (k >> 1) + 16 * (k & 1);
}

/* signs: int8 [rows, cols] of -1/+1 ; out: uint32 [rows, ceil(cols/32)] */
void nqo_pack_rows(const int8_t* signs, int64_t rows, int64_t cols, int half2, uint32_t* out) {
    int64_t words = (cols + 31) / 32;
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t w = 0; w < words; ++w) {
            uint32_t acc = 0;
            for (int k = 0; k < 32; ++k) {
                int64_t c = w * 32 + k;
                int8_t s = (c < cols) ? signs[r * cols + c] : (int8_t)1;
                if (s < 0) acc |= (uint32_t)1u << nqo_bit_position(k, half2);
            }
            out[r * words + w] = acc;
        }
    }
}

void nqo_unpack_rows(const uint32_t* packed, int64_t rows, int64_t cols, int half2, int8_t* out) {
    int64_t words = (cols + 31) / 32;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            uint32_t w = packed[r * words + c / 32];
            int bit = (w >> nqo_bit_position((int)(c % 32), half2)) & 1u;
            out[r * cols + c] = bit ? (int8_t)-1 : (int8_t)1;
        }
}

/* x [B,n], s_in [n], vt_bits [r, ceil(n/32)], s_mid [r] or NULL, u_bits [m, ceil(r/32)],
 * s_out [m] -> y [B,m]; all floating inputs/outputs are double. */
int nqo_layer_forward_packed(const double* x, const double* s_in, const uint32_t* vt_bits,
                             const double* s_mid, const uint32_t* u_bits, const double* s_out,
                             int64_t B, int64_t n, int64_t r, int64_t m, int half2, double* y) {
    int64_t wn = (n + 31) / 32, wr = (r + 31) / 32;
    double* h = (double*)malloc(sizeof(double) * (size_t)r);
    if (!h) return -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t i = 0; i < r; ++i) {
            double acc = 0.0;
            for (int64_t c = 0; c < n; ++c) {
                uint32_t w = vt_bits[i * wn + c / 32];
                double v = x[b * n + c] * s_in[c];
                acc += ((w >> nqo_bit_position((int)(c % 32), half2)) & 1u) ? -v : v;
            }
            h[i] = s_mid ? acc * s_mid[i] : acc;
        }
        for (int64_t j = 0; j < m; ++j) {
            double acc = 0.0;
            for (int64_t i = 0; i < r; ++i) {
                uint32_t w = u_bits[j * wr + i / 32];
                acc += ((w >> nqo_bit_position((int)(i % 32), half2)) & 1u) ? -h[i] : h[i];
            }
            y[b * m + j] = acc * s_out[j];
        }
    }
    free(h);
    return 0;
}
