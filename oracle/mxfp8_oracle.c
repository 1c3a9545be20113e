/* Scalar C restatement of the MXFP8 formats, the 32-block quantiser and the routed
 * FFN forward.  TEST INFRASTRUCTURE ONLY: an independent second implementation that
 * the numpy oracle is checked against (different arithmetic: frexp/nearbyint here, bit
 * tricks there).  Follows the same reference lines as oracle/moe_ffn.py:
 *   campaigns/mok/port/gemm/gemm.cu:150-162          (which operand is which)
 *   campaigns/mok/port/act_gptoss/swiglu.cuh:157-177 (activation, bf16 rounding)
 *   campaigns/mok/host/act_gptoss_reference.py:16-21 (activation closed form)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>

float plko_e4m3_decode(uint8_t c) {
  int e = (c >> 3) & 15, m = c & 7;
  float s = (c & 0x80) ? -1.0f : 1.0f;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) return s * ldexpf((float)m, -9);
  return s * ldexpf(1.0f + (float)m / 8.0f, e - 7);
}

uint8_t plko_e4m3_encode(float x) {
  uint8_t sign = signbit(x) ? 0x80 : 0;
  if (isnan(x)) return sign | 0x7F;
  float a = fabsf(x);
  if (a > 448.0f) a = 448.0f;
  if (a == 0.0f) return sign;
  int ex;
  float fr = frexpf(a, &ex); /* a = fr * 2^ex, fr in [0.5,1) */
  int e = ex - 1;            /* a = (2 fr) * 2^e, 2fr in [1,2) */
  if (e < -6) {              /* subnormal grid 2^-9 */
    int q = (int)nearbyintf(ldexpf(a, 9));
    return sign | (uint8_t)q; /* q == 8 is the first normal code */
  }
  int q = (int)nearbyintf(ldexpf(fr, 4)); /* 2fr*8 in [8,16] */
  if (q == 16) { q = 8; e += 1; }
  int code = ((e + 7) << 3) | (q - 8);
  if (code > 0x7E) code = 0x7E;
  return sign | (uint8_t)code;
}

float plko_e8m0_decode(uint8_t b) { return b == 255 ? NAN : (float)ldexp(1.0, (int)b - 127); }

uint8_t plko_e8m0_from_amax(float amax) {
  if (!(amax >= 1.17549435e-38f)) return 0; /* zero or subnormal */
  int ex;
  frexpf(amax, &ex); /* floor(log2) = ex-1 */
  int b = (ex - 1) - 8 + 127;
  if (b < 0) b = 0;
  if (b > 254) b = 254;
  return (uint8_t)b;
}

/* x [rows,k] f32 -> q [rows,k] u8, sc [rows,ld] u8 (ld >= k/32) */
void plko_mx_quantize(const float* x, long rows, long k, long ld, uint8_t* q, uint8_t* sc) {
  for (long r = 0; r < rows; ++r) {
    memset(sc + r * ld, 0, (size_t)ld);
    for (long b = 0; b < k / 32; ++b) {
      const float* v = x + r * k + b * 32;
      float amax = 0.0f;
      for (int i = 0; i < 32; ++i) { float a = fabsf(v[i]); if (a > amax) amax = a; }
      uint8_t sb = plko_e8m0_from_amax(amax);
      sc[r * ld + b] = sb;
      for (int i = 0; i < 32; ++i)
        q[r * k + b * 32 + i] = plko_e4m3_encode((float)ldexp((double)v[i], 127 - (int)sb));
    }
  }
}

float plko_bf16_round(float x) {
  uint32_t u; memcpy(&u, &x, 4);
  if (isnan(x)) return x;
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  float y; memcpy(&y, &u, 4); return y;
}

float plko_swiglu(float g, float u, float limit, int clamped) {
  if (clamped) { g = fminf(g, limit); u = fminf(fmaxf(u, -limit), limit); }
  float sig = 1.0f / (1.0f + expf(-1.702f * g));
  return (u + 1.0f) * (g * sig);
}

static void deq_row(const uint8_t* q, const uint8_t* sc, long k, float* out) {
  for (long i = 0; i < k; ++i) out[i] = plko_e4m3_decode(q[i]) * plko_e8m0_decode(sc[i / 32]);
}

/* out[r, n] = sum_k deq(a[arow(r)]) * deq(w[e][n]); rows grouped by expert; f32 accumulate in k order */
static void grouped(const uint8_t* aq, const uint8_t* asc, const int32_t* arow, long k, long ld,
                    const uint8_t* wq, const uint8_t* wsc, long n, const int32_t* counts, int ne, float* out) {
  float* ar = (float*)malloc(sizeof(float) * (size_t)k);
  float* wr = (float*)malloc(sizeof(float) * (size_t)k);
  long r = 0;
  for (int e = 0; e < ne; ++e)
    for (int c = 0; c < counts[e]; ++c, ++r) {
      long src = arow ? arow[r] : r;
      deq_row(aq + src * k, asc + src * ld, k, ar);
      for (long j = 0; j < n; ++j) {
        deq_row(wq + ((long)e * n + j) * k, wsc + ((long)e * n + j) * ld, k, wr);
        double s = 0.0;
        for (long i = 0; i < k; ++i) s += (double)ar[i] * (double)wr[i];
        out[r * n + j] = (float)s;
      }
    }
  free(ar); free(wr);
}

/* Full routed forward for small shapes.  H = d_model, I = d_ff.  y f32 (bf16-rounded) [R,H],
 * hq [R,I], hsc [R,ldi]. */
void plko_moe_forward(const uint8_t* xq, const uint8_t* xsc, const int32_t* row_token,
                      const uint8_t* wgq, const uint8_t* wgsc, const uint8_t* wuq, const uint8_t* wusc,
                      const uint8_t* wdq, const uint8_t* wdsc, const int32_t* counts, int ne,
                      long H, long I, long ldh, long ldi, float limit, int clamped,
                      float* y, uint8_t* hq, uint8_t* hsc) {
  long R = 0; for (int e = 0; e < ne; ++e) R += counts[e];
  float* gate = (float*)malloc(sizeof(float) * (size_t)(R * I));
  float* up = (float*)malloc(sizeof(float) * (size_t)(R * I));
  grouped(xq, xsc, row_token, H, ldh, wgq, wgsc, I, counts, ne, gate);
  grouped(xq, xsc, row_token, H, ldh, wuq, wusc, I, counts, ne, up);
  for (long i = 0; i < R * I; ++i) gate[i] = plko_bf16_round(plko_swiglu(gate[i], up[i], limit, clamped));
  plko_mx_quantize(gate, R, I, ldi, hq, hsc);
  grouped(hq, hsc, NULL, I, ldi, wdq, wdsc, H, counts, ne, y);
  for (long i = 0; i < R * H; ++i) y[i] = plko_bf16_round(y[i]);
  free(gate); free(up);
}
