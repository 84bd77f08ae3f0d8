/* CPU restatement (plain C, float32) of the reference's scan and pooling kernels.
 * TEST INFRASTRUCTURE ONLY: used by tests and by the CPU-baseline leg of the benchmark,
 * never by the shipped package.
 *
 * Each function follows the arithmetic order of the reference kernel it cites
 * (paths relative to /root/reference/code/libs/kangaroo/kangaroo_smat):
 *   orc_corr1ord          corr1ord.cuh:139-157   (j ascending, sequential float adds)
 *   orc_corr1ord_bprop_W  corr1ord_bprop.cuh:91-137 (the reference uses float atomics, so its
 *                          order is undefined; here positions are summed in ascending order)
 *   orc_corr1ord_bprop_X  corr1ord_bprop.cu:191-201 (the reference's own host loop)
 *   orc_poolrgn           poolrgn.cuh:44-160
 *   orc_poolrgn_bprop     poolrgn_bprop.cuh:45-127
 *   orc_scanpool          the same scan followed by bias, ReLU and pooling without storing the map
 * Pinned by tests/test_oracle_c.py against the NumPy oracle (itself pinned by closed forms).
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

enum { PT_MAX = 0, PT_AVG = 1, PT_SUM = 2, PT_ALL = 3 };

static inline float tapval(const float* W, size_t F, size_t j, unsigned k, size_t f)
{
    if (k < 4) return W[(4 * j + k) * F + f];
    if (k == 254) return 0.0f;
    float z = W[(4 * j) * F + f];
    z += W[(4 * j + 1) * F + f];
    z += W[(4 * j + 2) * F + f];
    z += W[(4 * j + 3) * F + f];
    return z * 0.25f;
}

/* Z[i,f] for i < n = N-m+1; rows >= n untouched. */
void orc_corr1ord(const float* W, size_t m, size_t F, const uint8_t* X, size_t N, float* Z)
{
    if (N + 1 < m + 1) return;
    size_t n = N - m + 1;
    #pragma omp parallel for schedule(static)
    for (long long ii = 0; ii < (long long)n; ++ii) {
        size_t i = (size_t)ii;
        for (size_t f = 0; f < F; ++f) {
            float z = 0.0f;
            for (size_t j = 0; j < m; ++j)
                z += tapval(W, F, j, X[i + j], f);
            Z[i * F + f] = z;
        }
    }
}

void orc_corr1ord_bprop_W(float* dW, size_t m, size_t F, const uint8_t* X, size_t N, const float* dZ)
{
    if (N + 1 < m + 1) return;
    size_t n = N - m + 1;
    for (size_t i = 0; i < n; ++i)
        for (size_t j = 0; j < m; ++j) {
            unsigned k = X[i + j];
            if (k < 4) {
                for (size_t f = 0; f < F; ++f) dW[(4 * j + k) * F + f] += dZ[i * F + f];
            } else if (k != 254) {
                for (size_t f = 0; f < F; ++f) {
                    float z = dZ[i * F + f] * 0.25f;
                    for (unsigned c = 0; c < 4; ++c) dW[(4 * j + c) * F + f] += z;
                }
            }
        }
}

void orc_corr1ord_bprop_X(float* dX, size_t n, const float* W, size_t m, size_t F, const float* dZ)
{
    for (size_t i = 0; i < n; ++i)
        for (size_t f = 0; f < F; ++f)
            for (size_t k = 0; k < m; ++k) {
                if (i < k) continue;
                for (size_t c = 0; c < 4; ++c)
                    dX[i * 4 + c] += dZ[(i - k) * F + f] * W[(4 * k + c) * F + f];
            }
}

void orc_poolrgn(const float* U, size_t F, const uint32_t* R, size_t P, int per_region_step,
                 float* pooled, uint32_t* argmax, int ptype)
{
    size_t rc = per_region_step ? 3 : 2;
    for (size_t r = 0; r < P; ++r) {
        size_t a = R[r * rc], b = R[r * rc + 1];
        size_t step = per_region_step ? R[r * rc + 2] : 1;
        size_t cnt = (b - a + step - 1) / step;
        for (size_t f = 0; f < F; ++f) {
            float x = U[a * F + f];
            float y = x;
            size_t xi = a * F + f;
            for (size_t i = a + step; i < b; i += step) {
                float v = U[i * F + f];
                if (v > x) { x = v; xi = i * F + f; }
                y += v;
            }
            if (ptype == PT_MAX) {
                pooled[r * F + f] = x;
            } else if (ptype == PT_SUM) {
                pooled[r * F + f] = y;
            } else if (ptype == PT_AVG) {
                pooled[r * F + f] = y / (float)cnt;
            } else {
                pooled[(r * F + f) * 2] = x;
                pooled[(r * F + f) * 2 + 1] = y / (float)cnt;
            }
            if (argmax && (ptype == PT_MAX || ptype == PT_ALL)) argmax[r * F + f] = (uint32_t)xi;
        }
    }
}

void orc_poolrgn_bprop(float* dU, size_t F, const uint32_t* R, size_t P, int per_region_step,
                       const float* dP, const uint32_t* argmax, int ptype)
{
    size_t rc = per_region_step ? 3 : 2;
    for (size_t r = 0; r < P; ++r) {
        size_t a = R[r * rc], b = R[r * rc + 1];
        size_t step = per_region_step ? R[r * rc + 2] : 1;
        size_t cnt = (b - a + step - 1) / step;
        for (size_t f = 0; f < F; ++f) {
            if (ptype == PT_MAX) {
                dU[argmax[r * F + f]] += dP[r * F + f];
            } else if (ptype == PT_ALL) {
                float dy = dP[(r * F + f) * 2 + 1] / (float)cnt;
                for (size_t i = a; i < b; i += step) dU[i * F + f] += dy;
                dU[argmax[r * F + f]] += dP[(r * F + f) * 2];
            } else {
                float v = dP[r * F + f];
                if (ptype == PT_AVG) v /= (float)cnt;
                for (size_t i = a; i < b; i += step) dU[i * F + f] += v;
            }
        }
    }
}

/* scan -> +bias -> ReLU -> pool over 2-column regions, never storing the (N,F) map.
 * pooled: (P,F) for max/avg, (P,2F) interleaved (max,avg) for all. argmax optional. */
void orc_scanpool(const float* W, const float* bias, size_t m, size_t F, const uint8_t* X, size_t N,
                  const uint32_t* R, size_t P, int ptype, float* pooled, uint32_t* argmax)
{
    #pragma omp parallel for schedule(dynamic, 16)
    for (long long rr = 0; rr < (long long)P; ++rr) {
        size_t r = (size_t)rr;
        size_t a = R[r * 2], b = R[r * 2 + 1];
        for (size_t f = 0; f < F; ++f) {
            float mx = 0.0f, sum = 0.0f;
            size_t xi = 0;
            for (size_t i = a; i < b; ++i) {
                float z = 0.0f;
                if (i + m <= N)
                    for (size_t j = 0; j < m; ++j) z += tapval(W, F, j, X[i + j], f);
                z += bias[f];
                z = z > 0.0f ? z : 0.0f;
                if (i == a || z > mx) { mx = z; xi = i * F + f; }
                sum = (i == a) ? z : sum + z;
            }
            float cnt = (float)(b - a);
            if (ptype == PT_MAX) pooled[r * F + f] = mx;
            else if (ptype == PT_AVG) pooled[r * F + f] = sum / cnt;
            else if (ptype == PT_SUM) pooled[r * F + f] = sum;
            else { pooled[(r * F + f) * 2] = mx; pooled[(r * F + f) * 2 + 1] = sum / cnt; }
            if (argmax && (ptype == PT_MAX || ptype == PT_ALL)) argmax[r * F + f] = (uint32_t)xi;
        }
    }
}
