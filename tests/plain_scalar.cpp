// A plain scalar 32-bit Llama decoder written from the reference's formulas, one function for each
// part, whole sequences, no cache, no paging, std::fma where the reference fuses and separate
// operations where it does not.  The engine's 32-bit path must give these bits.  It shares no code
// with the engine; it is compiled for the CPU by the tests (g++ -O2 -ffp-contract=off).
// Citations are file:line of the reference.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace {

// exp(x) as the engine's 32-bit path defines it (the reference calls libm's expf, src/kernels.cpp:328,
// whose bits differ between machines): k = rint(x * log2e), r = x - k ln2 with ln2 in two parts,
// the Taylor polynomial of degree 7 in Horner form, the result scaled by 2^k in two exact steps;
// below -87: 0, above 89: +inf, NaN stays NaN.
float ps_expf(float x) {
  if (!(x >= -87.0f)) return (x != x) ? x : 0.0f;
  if (x > 89.0f) return std::numeric_limits<float>::infinity();
  const float kf = std::nearbyintf(x * 0x1.715476p+0f);        // round to nearest, ties to even
  float r = std::fmaf(kf, -0x1.62e4p-1f, x);
  r = std::fmaf(kf, -0x1.7f7d1cp-20f, r);
  float p = 0x1.a01a02p-13f;                                    // 1/5040
  p = std::fmaf(p, r, 0x1.6c16c2p-10f);                         // 1/720
  p = std::fmaf(p, r, 0x1.111112p-7f);                          // 1/120
  p = std::fmaf(p, r, 0x1.555556p-5f);                          // 1/24
  p = std::fmaf(p, r, 0x1.555556p-3f);                          // 1/6
  p = std::fmaf(p, r, 0.5f);
  p = std::fmaf(p, r, 1.0f);
  p = std::fmaf(p, r, 1.0f);
  const int k = (int)kf;
  const int k1 = k >> 1, k2 = k - k1;
  return (p * std::ldexp(1.0f, k1)) * std::ldexp(1.0f, k2);
}

// 16 chains lane = i % 16, then the fixed tree (src/kernels.cpp:57-64, :86-101; spelled out in
// tests/test_main.cpp:126-131).
float ps_dot_canonical(const float* a, const float* b, int n) {
  float lane[16];
  for (int i = 0; i < 16; ++i) lane[i] = 0.0f;
  for (int i = 0; i < n; ++i) lane[i % 16] = std::fmaf(a[i], b[i], lane[i % 16]);
  float s8[8], s4[4];
  for (int i = 0; i < 8; ++i) s8[i] = lane[i] + lane[i + 8];
  for (int i = 0; i < 4; ++i) s4[i] = s8[i] + s8[i + 4];
  return (s4[0] + s4[2]) + (s4[1] + s4[3]);
}

// inv = 1/sqrt(sumsq/dim + eps); y = (x*inv)*w (src/kernels.cpp:264-271).
void ps_rmsnorm(const float* x, const float* w, float* y, int rows, int dim, float eps) {
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (size_t)r * dim;
    const float ss = ps_dot_canonical(xr, xr, dim);
    const float inv = 1.0f / std::sqrt(ss / (float)dim + eps);
    for (int i = 0; i < dim; ++i) y[(size_t)r * dim + i] = (xr[i] * inv) * w[i];
  }
}

// acc = 0; acc = fma(x[m,k], W[n,k], acc) for k ascending (src/kernels.cpp:236-244); no bias here.
void ps_linear(const float* x, const float* w, float* y, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) acc = std::fmaf(x[(size_t)m * K + k], w[(size_t)n * K + k], acc);
      y[(size_t)m * N + n] = acc;
    }
}

// Rotate-half pairs (i, i + hd/2): v[i] = x1*c - x2*s, v[i+hd/2] = x2*c + x1*s, separate multiplications
// and one subtraction or addition (src/kernels.cpp:273-289).  cos and sin of the row's position come from
// tables [position][hd/2] that the caller built on the host.
void ps_rope(float* v, int heads, int hd, const float* c, const float* s) {
  const int half = hd / 2;
  for (int h = 0; h < heads; ++h) {
    float* p = v + (size_t)h * hd;
    for (int i = 0; i < half; ++i) {
      const float x1 = p[i], x2 = p[i + half];
      const float a = x1 * c[i], b = x2 * s[i];
      const float d = x2 * c[i], e = x1 * s[i];
      p[i] = a - b;
      p[i + half] = d + e;
    }
  }
}

// One query against keys lo..pos of its kv head, two passes in key order (src/kernels.cpp:312-338):
// s_j = dot_canonical(q, k_j) * scale, the maximum from -inf; then e = exp(s_j - mx), sum += e,
// acc[d] = fma(e, v_j[d], acc[d]); out[d] = acc[d] * (1/sum).  k, v: [T][kv_heads][hd].
void ps_attend(const float* q, const float* k, const float* v, int kv_heads, int kvh, int hd, int lo, int pos,
               float scale, float* out) {
  float mx = -std::numeric_limits<float>::infinity();
  std::vector<float> sc(pos - lo + 1);
  for (int j = lo; j <= pos; ++j) {
    const float s = ps_dot_canonical(q, k + ((size_t)j * kv_heads + kvh) * hd, hd) * scale;
    sc[j - lo] = s;
    mx = s > mx ? s : mx;
  }
  std::vector<float> acc(hd, 0.0f);
  float sum = 0.0f;
  for (int j = lo; j <= pos; ++j) {
    const float e = ps_expf(sc[j - lo] - mx);
    sum += e;
    const float* vj = v + ((size_t)j * kv_heads + kvh) * hd;
    for (int d = 0; d < hd; ++d) acc[d] = std::fmaf(e, vj[d], acc[d]);
  }
  const float inv = 1.0f / sum;
  for (int d = 0; d < hd; ++d) out[d] = acc[d] * inv;
}

// h = g * (1/(1+exp(-g))) * u, left to right (src/kernels.cpp:291-298).
float ps_swiglu_one(float g, float u) { return g * (1.0f / (1.0f + ps_expf(-g))) * u; }

}  // namespace

extern "C" {

void plain_expf(const float* x, float* y, long long n) {
  for (long long i = 0; i < n; ++i) y[i] = ps_expf(x[i]);
}

void plain_swiglu(const float* gate, const float* up, float* h, long long n) {
  for (long long i = 0; i < n; ++i) h[i] = ps_swiglu_one(gate[i], up[i]);
}

void plain_linear(const float* x, const float* w, float* y, int M, int N, int K) { ps_linear(x, w, y, M, N, K); }

void plain_rmsnorm(const float* x, const float* w, float* y, int rows, int dim, float eps) {
  ps_rmsnorm(x, w, y, rows, dim, eps);
}

float plain_dot_canonical(const float* a, const float* b, int n) { return ps_dot_canonical(a, b, n); }

// Causal grouped-query attention over one whole sequence: q [T][heads][hd], k and v [T][kv_heads][hd]
// (rotated already), head h reads kv head h / (heads / kv_heads) (src/kernels.cpp:342-368);
// scale = 1/sqrt(hd) (:347).  window 0: all keys; else keys pos-window+1..pos.
void plain_attention(const float* q, const float* k, const float* v, float* out, int T, int heads, int kv_heads, int hd,
                     int window) {
  const float scale = 1.0f / std::sqrt((float)hd);
  const int group = heads / kv_heads;
  for (int p = 0; p < T; ++p)
    for (int h = 0; h < heads; ++h) {
      const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
      ps_attend(q + ((size_t)p * heads + h) * hd, k, v, kv_heads, h / group, hd, lo, p, scale,
                out + ((size_t)p * heads + h) * hd);
    }
}

// The whole decoder over one sequence, every position's logits (src/model.cpp:267-322 with every row wanted).
// weights: one blob of floats in this order: embedding [V,H]; per layer input norm [H], q [QD,H], k [KVD,H],
// v [KVD,H], o [H,QD], post-attention norm [H], gate [I,H], up [I,H], down [H,I]; final norm [H]; head [V,H].
// cos, sin: [positions][hd/2] for positions first_position .. first_position + T - 1 at rows 0 .. T-1.
// windows: per layer, the number of keys a query sees (0: all; the reference has no window).
void plain_forward(const float* weights, const int32_t* tokens, int T, int V, int H, int L, int heads, int kv_heads,
                   int hd, int I, float eps, const int32_t* windows, const float* cos_rows, const float* sin_rows,
                   float* logits) {
  const int QD = heads * hd, KVD = kv_heads * hd, half = hd / 2;
  const float* embed = weights;
  const float* at = weights + (size_t)V * H;
  std::vector<float> x((size_t)T * H), xn((size_t)T * H), q((size_t)T * QD), k((size_t)T * KVD), v((size_t)T * KVD),
      attn((size_t)T * QD), proj((size_t)T * H), gate((size_t)T * I), up((size_t)T * I), hmid((size_t)T * I);
  for (int r = 0; r < T; ++r)                                            // src/model.cpp:274
    std::memcpy(&x[(size_t)r * H], embed + (size_t)tokens[r] * H, sizeof(float) * H);
  for (int l = 0; l < L; ++l) {
    const float* n1 = at;            at += H;
    const float* wq = at;            at += (size_t)QD * H;
    const float* wk = at;            at += (size_t)KVD * H;
    const float* wv = at;            at += (size_t)KVD * H;
    const float* wo = at;            at += (size_t)H * QD;
    const float* n2 = at;            at += H;
    const float* wg = at;            at += (size_t)I * H;
    const float* wu = at;            at += (size_t)I * H;
    const float* wd = at;            at += (size_t)H * I;
    ps_rmsnorm(x.data(), n1, xn.data(), T, H, eps);                      // :281
    ps_linear(xn.data(), wq, q.data(), T, QD, H);                        // :282 (the stacked product, side by side)
    ps_linear(xn.data(), wk, k.data(), T, KVD, H);
    ps_linear(xn.data(), wv, v.data(), T, KVD, H);
    for (int r = 0; r < T; ++r) {                                        // :289-290
      ps_rope(&q[(size_t)r * QD], heads, hd, cos_rows + (size_t)r * half, sin_rows + (size_t)r * half);
      ps_rope(&k[(size_t)r * KVD], kv_heads, hd, cos_rows + (size_t)r * half, sin_rows + (size_t)r * half);
    }
    plain_attention(q.data(), k.data(), v.data(), attn.data(), T, heads, kv_heads, hd, windows[l]);   // :298
    ps_linear(attn.data(), wo, proj.data(), T, H, QD);                   // :299
    for (size_t i = 0; i < (size_t)T * H; ++i) x[i] += proj[i];          // :300
    ps_rmsnorm(x.data(), n2, xn.data(), T, H, eps);                      // :301
    ps_linear(xn.data(), wg, gate.data(), T, I, H);                      // :302
    ps_linear(xn.data(), wu, up.data(), T, I, H);
    for (size_t i = 0; i < (size_t)T * I; ++i) hmid[i] = ps_swiglu_one(gate[i], up[i]);   // :303
    ps_linear(hmid.data(), wd, proj.data(), T, H, I);                    // :304
    for (size_t i = 0; i < (size_t)T * H; ++i) x[i] += proj[i];          // :305
  }
  const float* nf = at;              at += H;
  const float* head = at;
  ps_rmsnorm(x.data(), nf, xn.data(), T, H, eps);                        // :318
  ps_linear(xn.data(), head, logits, T, V, H);                           // :319-320
}

}  // extern "C"
