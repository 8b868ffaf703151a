/*
 * Brute-force triple-loop evaluation of the two grouped GEMMs (test infrastructure, see
 * oracle/__init__.py).  It exists to pin the vectorised numpy oracle: it shares no code with it
 * and follows the per-expert pointer arithmetic of the reference literally
 * (expert_specialization/csrc/cuda/es_fp8_blockwise_functor.cuh:57-74,
 *  expert_specialization/csrc/cuda/es_sm100_mxfp8_blockscaled_functor.cuh:61-75).
 * Results are double precision (no output rounding).
 */
#include <math.h>
#include <stdint.h>

static double e4m3fn(uint8_t b) {
  int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
  double v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexp(m / 8.0, -6);
  else v = ldexp(1.0 + m / 8.0, e - 7);
  return s ? -v : v;
}

/* out[off_e + m][n] = sum_k (sa[off_e+m][k/128] * a[off_e+m][k]) * (sb[e][n/128][k/128] * b[e][n][k]) */
void brute_fp8_blockwise(const uint8_t* a, const uint8_t* b, const float* sa, const float* sb, const int32_t* ps,
                         const int32_t* eo, int num_experts, double* out) {
  for (int e = 0; e < num_experts; e++) {
    int m_e = ps[3 * e], n = ps[3 * e + 1], k = ps[3 * e + 2];
    int64_t off = eo[e];
    const uint8_t* a_e = a + off * k;
    const uint8_t* b_e = b + (int64_t)e * k * n;
    const float* sa_e = sa + off * k / 128;
    const float* sb_e = sb + (int64_t)e * k * n / 128 / 128;
    double* out_e = out + off * n;
    for (int m = 0; m < m_e; m++)
      for (int j = 0; j < n; j++) {
        double acc = 0;
        for (int kk = 0; kk < k; kk++) {
          double av = (double)sa_e[(int64_t)m * (k / 128) + kk / 128] * e4m3fn(a_e[(int64_t)m * k + kk]);
          double bv = (double)sb_e[(int64_t)(j / 128) * (k / 128) + kk / 128] * e4m3fn(b_e[(int64_t)j * k + kk]);
          acc += av * bv;
        }
        out_e[(int64_t)m * n + j] = acc;
      }
  }
}

/* byte offset of scale (row r, scale column c) inside one expert's block of swizzled 128x4 tiles,
 * written as the CuTe layout ((32,4),4):((16,4),1) tiled K-fastest
 * (es_sm100_mxfp8_blockscaled_group_quant.cuh:25,294-307) */
int64_t brute_sf_offset(int r, int c, int k) {
  int tile_m = r / 128, tile_k = c / 4;
  int r_in = r % 128, c_in = c % 4;
  int i0 = r_in % 32, i1 = r_in / 32; /* shape (32,4) stride (16,4) */
  return ((int64_t)tile_m * (k / 128) + tile_k) * 512 + i0 * 16 + i1 * 4 + c_in;
}

void brute_mxfp8(const uint8_t* a, const uint8_t* b, const uint8_t* sfa, const uint8_t* sfb, const int32_t* ps,
                 const int32_t* eo, const int32_t* bso, int num_experts, double* out) {
  for (int e = 0; e < num_experts; e++) {
    int m_e = ps[3 * e], n = ps[3 * e + 1], k = ps[3 * e + 2];
    int64_t off = eo[e];
    const uint8_t* a_e = a + off * k;
    const uint8_t* b_e = b + (int64_t)e * k * n;
    const uint8_t* sfa_e = sfa + (int64_t)bso[e] * (k / 32);
    const uint8_t* sfb_e = sfb + (int64_t)e * n * (k / 32);
    double* out_e = out + off * n;
    for (int m = 0; m < m_e; m++)
      for (int j = 0; j < n; j++) {
        double acc = 0;
        for (int kk = 0; kk < k; kk++) {
          double av = ldexp(e4m3fn(a_e[(int64_t)m * k + kk]), (int)sfa_e[brute_sf_offset(m, kk / 32, k)] - 127);
          double bv = ldexp(e4m3fn(b_e[(int64_t)j * k + kk]), (int)sfb_e[brute_sf_offset(j, kk / 32, k)] - 127);
          acc += av * bv;
        }
        out_e[(int64_t)m * n + j] = acc;
      }
  }
}
