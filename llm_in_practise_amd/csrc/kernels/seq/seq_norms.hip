// Token-wise kernels of models that keep their residual stream in float: scaled embedding with sinusoidal
// positions, RMS norms that read float and write the activation type, the gated + normed residual update
// (fused with the next sublayer's entry norm), the mean of two normed branches, PolyNorm, and the per-head
// norm + output gate that follows a recurrent mixer.  One 256-thread block per token (one wave per head for the
// head norm); rows are re-read for the second pass (they sit in L1/L2), so any width works.
#include "seq_common.h"

using namespace lipa;

// x[t, c] = table[tok[t], c] * scale + (c even ? sin : cos)(pos[t] * inv_freq[c / 2])
template <typename T>
__global__ __launch_bounds__(256) void k_embed_sincos(const long* __restrict__ tok, const int* __restrict__ pos,
                                                      const T* __restrict__ table, const float* __restrict__ inv_freq,
                                                      float* __restrict__ x, int W, float scale) {
  const int t = blockIdx.x;
  const long id = tok[t];
  const float p = (float)pos[t];
  for (int c = threadIdx.x; c < W; c += 256) {
    const float a = p * inv_freq[c >> 1];
    x[(size_t)t * W + c] = (float)table[(size_t)id * W + c] * scale + ((c & 1) ? cosf(a) : sinf(a));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void k_rms_f32(const float* __restrict__ x, const float* __restrict__ w,
                                                 T* __restrict__ out, int W, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) { const float v = x[r + c]; s += v * v; }
  const float rs = rsqrtf(block_sum256(s, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) out[r + c] = (T)(x[r + c] * rs * w[c]);
}

// z = y * sigmoid(r + b);  x += z / rms(z) * wb;  optionally h = x / rms(x) * wn
template <typename T>
__global__ __launch_bounds__(256) void k_gated_residual(float* __restrict__ x, const T* __restrict__ y, int ldy,
                                                        const T* __restrict__ r, int ldr, const float* __restrict__ b,
                                                        const float* __restrict__ wb, const float* __restrict__ wn,
                                                        T* __restrict__ h, int W, float eps) {
  __shared__ float sc[4];
  const size_t t = blockIdx.x;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float z = (float)y[t * ldy + c] * sigmoidf_((float)r[t * ldr + c] + b[c]);
    s += z * z;
  }
  const float rs = rsqrtf(block_sum256(s, sc) / W + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float z = (float)y[t * ldy + c] * sigmoidf_((float)r[t * ldr + c] + b[c]);
    const float v = x[t * W + c] + z * rs * wb[c];
    x[t * W + c] = v;
    s2 += v * v;
  }
  if (wn == nullptr) return;
  const float rs2 = rsqrtf(block_sum256(s2, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256) h[t * W + c] = (T)(x[t * W + c] * rs2 * wn[c]);
}

// out = 0.5 * (a / rms(a) * wa + b / rms(b) * wb)
template <typename T>
__global__ __launch_bounds__(256) void k_dual_norm_mean(const T* __restrict__ a, const T* __restrict__ b,
                                                        const float* __restrict__ wa, const float* __restrict__ wb,
                                                        T* __restrict__ out, int W, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * W;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float u = (float)a[r + c], v = (float)b[r + c];
    sa += u * u;
    sb += v * v;
  }
  const float ra = rsqrtf(block_sum256(sa, sc) / W + eps);
  const float rb = rsqrtf(block_sum256(sb, sc) / W + eps);
  for (int c = threadIdx.x; c < W; c += 256)
    out[r + c] = (T)(0.5f * ((float)a[r + c] * ra * wa[c] + (float)b[r + c] * rb * wb[c]));
}

// PolyNorm: c0 z/rms(z) + c1 z^2/rms(z^2) + c2 z^3/rms(z^3) + c3 over a token's vector
template <typename T>
__global__ __launch_bounds__(256) void k_polynorm(const T* __restrict__ z, const float* __restrict__ coef,
                                                  T* __restrict__ out, int F, float eps) {
  __shared__ float sc[4];
  const size_t r = (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = (float)z[r + c], v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  const float r1 = coef[0] * rsqrtf(block_sum256(s1, sc) / F + eps);
  const float r2 = coef[1] * rsqrtf(block_sum256(s2, sc) / F + eps);
  const float r3 = coef[2] * rsqrtf(block_sum256(s3, sc) / F + eps);
  const float c3 = coef[3];
  for (int c = threadIdx.x; c < F; c += 256) {
    const float v = (float)z[r + c], v2 = v * v;
    out[r + c] = (T)(v * r1 + v2 * r2 + v2 * v * r3 + c3);
  }
}

// out[t, h, c] = o[t, h, c] / rms_c(o[t, h, :]) * w[(per_head ? h * dv : 0) + c] * sigmoid(gate[t, h * dv + c]);
// with den / efl (per token and head) o is first divided by max(|den|, efl) + 1e-6 (the mLSTM read-out)
template <typename T>
__global__ __launch_bounds__(256) void k_head_norm_gate(const float* __restrict__ o, const float* __restrict__ w,
                                                        int per_head, const T* __restrict__ gate, int ldg,
                                                        const float* __restrict__ den, const float* __restrict__ efl,
                                                        T* __restrict__ out, int nrows, int H, int dv, float eps) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= nrows) return;
  const int t = row / H, hd = row % H;
  const float* src = o + (size_t)row * dv;
  const float dinv = den != nullptr ? 1.f / (fmaxf(fabsf(den[row]), efl[row]) + 1e-6f) : 1.f;
  float s = 0.f;
  for (int c = lane; c < dv; c += 64) {
    const float v = src[c] * dinv;
    s += v * v;
  }
  const float rs = rsqrtf(wave_sum(s) / dv + eps) * dinv;
  for (int c = lane; c < dv; c += 64) {
    const float g = sigmoidf_((float)gate[(size_t)t * ldg + hd * dv + c]);
    out[(size_t)row * dv + c] = (T)(src[c] * rs * w[(per_head ? hd * dv : 0) + c] * g);
  }
}

// g = exp(-exp(A_log[h]) * softplus(pre + bias)), laid out [T, H * dk]
__global__ __launch_bounds__(256) void k_decay_gate(const float* __restrict__ pre, const float* __restrict__ bias,
                                                    const float* __restrict__ a_log, float* __restrict__ g, size_t n,
                                                    int HD, int dk) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int c = (int)(i % HD);
  g[i] = expf(-expf(a_log[c / dk]) * softplusf_(pre[i] + bias[c]));
}

// ---------------------------------------------------------------------------------------------- launchers
void seq_embed_sincos(int code, const long* tok, const int* pos, const void* table, const float* inv_freq, float* x,
                      int T_, int W, float scale, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_embed_sincos<T>, dim3(T_), dim3(256), 0, st, tok, pos, (const T*)table,
                                          inv_freq, x, W, scale));
  LIPA_CHECK_LAUNCH();
}

void seq_rms_f32(int code, const float* x, const float* w, void* out, int T_, int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_rms_f32<T>, dim3(T_), dim3(256), 0, st, x, w, (T*)out, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_gated_residual(int code, float* x, const void* y, int ldy, const void* r, int ldr, const float* b,
                        const float* wb, const float* wn, void* h, int T_, int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_gated_residual<T>, dim3(T_), dim3(256), 0, st, x, (const T*)y, ldy,
                                          (const T*)r, ldr, b, wb, wn, (T*)h, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_dual_norm_mean(int code, const void* a, const void* b, const float* wa, const float* wb, void* out, int T_,
                        int W, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_dual_norm_mean<T>, dim3(T_), dim3(256), 0, st, (const T*)a, (const T*)b,
                                          wa, wb, (T*)out, W, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_polynorm(int code, const void* z, const float* coef, void* out, int T_, int F, float eps, hipStream_t st) {
  if (T_ == 0) return;
  SEQ_DISPATCH_T(code,
                 hipLaunchKernelGGL(k_polynorm<T>, dim3(T_), dim3(256), 0, st, (const T*)z, coef, (T*)out, F, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_head_norm_gate(int code, const float* o, const float* w, int per_head, const void* gate, int ldg,
                        const float* den, const float* efl, void* out, int T_, int H, int dv, float eps, hipStream_t st) {
  const int rows = T_ * H;
  if (rows == 0) return;
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_head_norm_gate<T>, dim3((rows + 3) / 4), dim3(256), 0, st, o, w, per_head,
                                          (const T*)gate, ldg, den, efl, (T*)out, rows, H, dv, eps));
  LIPA_CHECK_LAUNCH();
}

void seq_decay_gate(const float* pre, const float* bias, const float* a_log, float* g, int T_, int HD, int dk,
                    hipStream_t st) {
  const size_t n = (size_t)T_ * HD;
  if (n == 0) return;
  hipLaunchKernelGGL(k_decay_gate, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, pre, bias, a_log, g, n, HD, dk);
  LIPA_CHECK_LAUNCH();
}
