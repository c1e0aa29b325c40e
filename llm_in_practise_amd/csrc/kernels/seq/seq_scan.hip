// Short causal convolutions with carried inputs, and the two matrix-memory recurrences (mLSTM with a running
// maximum; gated delta rule with a per-channel decay), over packed variable-length sequences with per-slot state.
//
// Recurrences: every column of the state matrix S[dk, dv] evolves on its own given the step's k, q and gates, so a
// block owns one (sequence, head) and up to 256/R columns; a column's dk rows are spread over R adjacent lanes
// (R a power of two <= 64, <= 16 rows per lane, rows interleaved i*R + rg) and live in registers for the whole
// scan.  Dot products over dk are finished with xor-shuffles inside the R-lane group: no barrier per token.  The
// step inputs of 16 tokens at a time are staged through LDS as float.  One token is the decode step: load state,
// one update, store.  State layout in HBM: S [slots, H, dv, dk] (a lane's rows are R apart, a group's lanes
// adjacent: coalesced), float.
#include "seq_common.h"

using namespace lipa;

constexpr int KR = 16;      // state rows per lane
constexpr int CT = 16;      // tokens staged per chunk
constexpr int MAXHW = 8;    // conv: head width <= 64 * MAXHW
constexpr int MAXTAPS = 8;

struct ConvSeg {
  int c0, nheads, hw, mode;   // mode 0: plain, 1: rms norm * w, 2: silu, 3: silu then unit vector * scale
  const float* w;
  float scale;
};
struct ConvArgs {
  ConvSeg seg[3];
  int nseg;
};

template <typename T>
__device__ __forceinline__ float conv_at(const T* __restrict__ u, int ldu, const T* __restrict__ state, int C, int taps,
                                         const float* __restrict__ w, int t, int j, int p0, int slot, int ch) {
  float acc = 0.f;
  for (int jj = 0; jj < taps; ++jj) {
    const int src = j - (taps - 1) + jj;
    float uv = 0.f;
    if (src >= 0)
      uv = (float)u[(size_t)(t - (taps - 1) + jj) * ldu + ch];
    else if (p0 > 0)
      uv = (float)state[((size_t)slot * (taps - 1) + (taps - 1 + src)) * C + ch];
    acc += w[(size_t)ch * taps + jj] * uv;
  }
  return acc;
}

// one wave per (token, head): convolution over time, then the head's activation / norm
template <typename T, typename OT>
__global__ __launch_bounds__(64) void k_short_conv(const T* __restrict__ u, int ldu, const float* __restrict__ w,
                                                   const T* __restrict__ state, OT* __restrict__ out, int C, int taps,
                                                   ConvArgs a, SeqDesc d, float eps) {
  const int t = blockIdx.x, lane = threadIdx.x;
  int hl = blockIdx.y, si = 0;
  while (si < a.nseg - 1 && hl >= a.seg[si].nheads) hl -= a.seg[si++].nheads;
  const ConvSeg sg = a.seg[si];
  const int s = d.tok_seq[t], j = t - d.seq_off[s], p0 = d.pos0[s], slot = d.slots[s];
  const int cbase = sg.c0 + hl * sg.hw;
  float vals[MAXHW];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXHW; ++i) {
    const int c = lane + 64 * i;
    vals[i] = 0.f;
    if (c < sg.hw) {
      float acc = conv_at(u, ldu, state, C, taps, w, t, j, p0, slot, cbase + c);
      if (sg.mode >= 2) acc = acc * sigmoidf_(acc);
      vals[i] = acc;
      ss += acc * acc;
    }
  }
  float mul = 1.f;
  if (sg.mode == 1) mul = rsqrtf(wave_sum(ss) / sg.hw + eps);
  if (sg.mode == 3) mul = rsqrtf(wave_sum(ss) + 1e-6f) * sg.scale;
#pragma unroll
  for (int i = 0; i < MAXHW; ++i) {
    const int c = lane + 64 * i;
    if (c < sg.hw) {
      float v = vals[i] * mul;
      if (sg.mode == 1) v *= sg.w[c];
      out[(size_t)t * C + cbase + c] = (OT)v;
    }
  }
}

// the last taps-1 inputs of every sequence become its carried state (older ones shift out)
template <typename T>
__global__ __launch_bounds__(256) void k_conv_state(const T* __restrict__ u, int ldu, T* __restrict__ state, int C,
                                                    int taps, SeqDesc d) {
  const int s = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
  if (ch >= C || (d.live && !d.live[s])) return;
  const int t0 = d.seq_off[s], len = d.seq_off[s + 1] - t0, p0 = d.pos0[s], slot = d.slots[s];
  float nv[MAXTAPS];
#pragma unroll
  for (int i = 0; i < MAXTAPS; ++i) {
    nv[i] = 0.f;
    if (i < taps - 1) {
      const int li = len - (taps - 1) + i;
      if (li >= 0)
        nv[i] = (float)u[(size_t)(t0 + li) * ldu + ch];
      else if (p0 > 0)
        nv[i] = (float)state[((size_t)slot * (taps - 1) + (taps - 1 + li)) * C + ch];
    }
  }
#pragma unroll
  for (int i = 0; i < MAXTAPS; ++i)
    if (i < taps - 1) state[((size_t)slot * (taps - 1) + i) * C + ch] = (T)nv[i];
}

__device__ __forceinline__ float group_sum(float v, int R) {
  for (int o = R >> 1; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// mLSTM.  m_t = max(f + m, i); S = e^(f+m-m_t) S + e^(i-m_t) k v^T; n likewise; o = S^T q / (max(|n.q|, e^-m_t) + 1e-6)
// with i = cap tanh((ipre + ib) / cap), f = logsigmoid(cap tanh((fpre + fb) / cap)); m starts at 0.
template <typename T>
__global__ __launch_bounds__(256) void k_mlstm_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                    const T* __restrict__ v, int ldv, const float* __restrict__ ipre,
                                                    const float* __restrict__ fpre, const float* __restrict__ ib,
                                                    const float* __restrict__ fb, float cap, float qscale,
                                                    float* __restrict__ S, float* __restrict__ N, float* __restrict__ M,
                                                    float* __restrict__ out, int H, int dk, int dv, int R, SeqDesc d) {
  extern __shared__ float smem[];
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int NC = 256 / R, rg = tid % R, cl = tid / R, col = cb * NC + cl;
  const bool colok = col < dv;
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  float* sk = smem;
  float* sq = sk + CT * dk;
  float* sv = sq + CT * dk;
  float* sg = sv + CT * NC;
  const size_t hbase = (size_t)slot * H + hd;
  float* Sp = S + (hbase * dv + (colok ? col : 0)) * dk;
  float Sr[KR], nr[KR];
  float m = p0 > 0 ? M[hbase] : 0.f;
#pragma unroll
  for (int i = 0; i < KR; ++i) {
    const int row = i * R + rg;
    Sr[i] = (p0 > 0 && colok && row < dk) ? Sp[row] : 0.f;
    nr[i] = (p0 > 0 && row < dk) ? N[hbase * dk + row] : 0.f;
  }
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
    for (int e = tid; e < n * dk; e += 256) {
      const int tt = e / dk, r = e % dk;
      sk[e] = (float)k[(size_t)(c0 + tt) * ldk + hd * dk + r];
      sq[e] = (float)q[(size_t)(c0 + tt) * ldq + hd * dk + r] * qscale;
    }
    for (int e = tid; e < n * NC; e += 256) {
      const int tt = e / NC, cc = cb * NC + e % NC;
      sv[e] = cc < dv ? (float)v[(size_t)(c0 + tt) * ldv + hd * dv + cc] : 0.f;
    }
    if (tid < n) {
      const float ip = ipre[(size_t)(c0 + tid) * H + hd] + ib[hd], fp = fpre[(size_t)(c0 + tid) * H + hd] + fb[hd];
      sg[2 * tid] = cap * tanhf(ip / cap);
      sg[2 * tid + 1] = logsigmoidf_(cap * tanhf(fp / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float ig = sg[2 * tt], fg = sg[2 * tt + 1];
      const float mn = fmaxf(fg + m, ig);
      const float a = expf(fg + m - mn), b = expf(ig - mn);
      m = mn;
      const float bv = b * sv[tt * NC + cl];
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int i = 0; i < KR; ++i) {
        const int row = i * R + rg;
        const bool ok = row < dk;
        const float kk = ok ? sk[tt * dk + row] : 0.f, qq = ok ? sq[tt * dk + row] : 0.f;
        Sr[i] = a * Sr[i] + kk * bv;
        nr[i] = a * nr[i] + b * kk;
        num += Sr[i] * qq;
        den += nr[i] * qq;
      }
      num = group_sum(num, R);
      den = group_sum(den, R);
      if (rg == 0 && colok)
        out[((size_t)(c0 + tt) * H + hd) * dv + col] = num / (fmaxf(fabsf(den), expf(-m)) + 1e-6f);
    }
  }
#pragma unroll
  for (int i = 0; i < KR; ++i) {
    const int row = i * R + rg;
    if (row < dk) {
      if (colok) Sp[row] = Sr[i];
      if (cb == 0 && cl == 0) N[hbase * dk + row] = nr[i];
    }
  }
  if (cb == 0 && tid == 0) M[hbase] = m;
}

// Gated delta rule.  S <- g * S (g per key channel); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
// beta = sigmoid(bpre); head hd reads q/k head hd / (H / G).
template <typename T>
__global__ __launch_bounds__(256) void k_delta_scan(const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk,
                                                    const T* __restrict__ v, int ldv, const float* __restrict__ g,
                                                    const float* __restrict__ bpre, float* __restrict__ S,
                                                    float* __restrict__ out, int H, int G, int dk, int dv, int R,
                                                    SeqDesc d) {
  extern __shared__ float smem[];
  const int s = blockIdx.x / H, hd = blockIdx.x % H, cb = blockIdx.y, tid = threadIdx.x;
  if (d.live && !d.live[s]) return;
  const int NC = 256 / R, rg = tid % R, cl = tid / R, col = cb * NC + cl, kh = hd / (H / G);
  const bool colok = col < dv;
  const int t0 = d.seq_off[s], t1 = d.seq_off[s + 1], p0 = d.pos0[s], slot = d.slots[s];
  float* sk = smem;
  float* sq = sk + CT * dk;
  float* sd = sq + CT * dk;
  float* sv = sd + CT * dk;
  float* sb = sv + CT * NC;
  float* Sp = S + (((size_t)slot * H + hd) * dv + (colok ? col : 0)) * dk;
  float Sr[KR];
#pragma unroll
  for (int i = 0; i < KR; ++i) {
    const int row = i * R + rg;
    Sr[i] = (p0 > 0 && colok && row < dk) ? Sp[row] : 0.f;
  }
  for (int c0 = t0; c0 < t1; c0 += CT) {
    const int n = min(CT, t1 - c0);
    __syncthreads();
    for (int e = tid; e < n * dk; e += 256) {
      const int tt = e / dk, r = e % dk;
      sk[e] = (float)k[(size_t)(c0 + tt) * ldk + kh * dk + r];
      sq[e] = (float)q[(size_t)(c0 + tt) * ldq + kh * dk + r];
      sd[e] = g[((size_t)(c0 + tt) * H + hd) * dk + r];
    }
    for (int e = tid; e < n * NC; e += 256) {
      const int tt = e / NC, cc = cb * NC + e % NC;
      sv[e] = cc < dv ? (float)v[(size_t)(c0 + tt) * ldv + hd * dv + cc] : 0.f;
    }
    if (tid < n) sb[tid] = sigmoidf_(bpre[(size_t)(c0 + tid) * H + hd]);
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < KR; ++i) {
        const int row = i * R + rg;
        if (row < dk) {
          Sr[i] *= sd[tt * dk + row];
          dot += Sr[i] * sk[tt * dk + row];
        }
      }
      dot = group_sum(dot, R);
      const float u = sb[tt] * (sv[tt * NC + cl] - dot);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < KR; ++i) {
        const int row = i * R + rg;
        if (row < dk) {
          Sr[i] += sk[tt * dk + row] * u;
          o += Sr[i] * sq[tt * dk + row];
        }
      }
      o = group_sum(o, R);
      if (rg == 0 && colok) out[((size_t)(c0 + tt) * H + hd) * dv + col] = o;
    }
  }
#pragma unroll
  for (int i = 0; i < KR; ++i) {
    const int row = i * R + rg;
    if (row < dk && colok) Sp[row] = Sr[i];
  }
}

// ---------------------------------------------------------------------------------------------- launchers
static int rows_split(int dk) {
  int R = 1;
  while (R * KR < dk) R <<= 1;
  return R;
}

int seq_scan_max_dk() { return 256; }   // 3 staged arrays of CT x dk floats stay under 64 KB of LDS
int seq_conv_max_head() { return 64 * MAXHW; }
int seq_conv_max_taps() { return MAXTAPS; }

// segs: nseg x {c0, nheads, hw, mode}; sw: nseg norm-weight pointers (or null); sscale: nseg scales
void seq_short_conv(int code, int out_f32, const void* u, int ldu, const float* w, void* state, void* out, int C,
                    int taps, int nseg, const int* segs, const float* const* sw, const float* sscale, SeqDesc d,
                    float eps, hipStream_t st) {
  if (d.Ttot == 0) return;
  ConvArgs a;
  a.nseg = nseg;
  int heads = 0;
  for (int i = 0; i < nseg; ++i) {
    a.seg[i] = ConvSeg{segs[4 * i], segs[4 * i + 1], segs[4 * i + 2], segs[4 * i + 3], sw[i], sscale[i]};
    heads += segs[4 * i + 1];
  }
  SEQ_DISPATCH_T(code, {
    if (out_f32)
      hipLaunchKernelGGL((k_short_conv<T, float>), dim3(d.Ttot, heads), dim3(64), 0, st, (const T*)u, ldu, w,
                         (const T*)state, (float*)out, C, taps, a, d, eps);
    else
      hipLaunchKernelGGL((k_short_conv<T, T>), dim3(d.Ttot, heads), dim3(64), 0, st, (const T*)u, ldu, w,
                         (const T*)state, (T*)out, C, taps, a, d, eps);
    if (taps > 1)
      hipLaunchKernelGGL(k_conv_state<T>, dim3(d.B, (C + 255) / 256), dim3(256), 0, st, (const T*)u, ldu, (T*)state, C,
                         taps, d);
  });
  LIPA_CHECK_LAUNCH();
}

void seq_mlstm_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* ipre,
                    const float* fpre, const float* ib, const float* fb, float cap, float qscale, float* S, float* N,
                    float* M, float* out, int H, int dk, int dv, SeqDesc d, hipStream_t st) {
  if (d.B == 0) return;
  const int R = rows_split(dk), NC = 256 / R;
  const size_t lds = sizeof(float) * ((size_t)2 * CT * dk + CT * NC + 2 * CT);
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_mlstm_scan<T>, dim3(d.B * H, (dv + NC - 1) / NC), dim3(256), lds, st,
                                          (const T*)q, ldq, (const T*)k, ldk, (const T*)v, ldv, ipre, fpre, ib, fb, cap,
                                          qscale, S, N, M, out, H, dk, dv, R, d));
  LIPA_CHECK_LAUNCH();
}

void seq_delta_scan(int code, const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* g,
                    const float* bpre, float* S, float* out, int H, int G, int dk, int dv, SeqDesc d, hipStream_t st) {
  if (d.B == 0) return;
  const int R = rows_split(dk), NC = 256 / R;
  const size_t lds = sizeof(float) * ((size_t)3 * CT * dk + CT * NC + CT);
  SEQ_DISPATCH_T(code, hipLaunchKernelGGL(k_delta_scan<T>, dim3(d.B * H, (dv + NC - 1) / NC), dim3(256), lds, st,
                                          (const T*)q, ldq, (const T*)k, ldk, (const T*)v, ldv, g, bpre, S, out, H, G,
                                          dk, dv, R, d));
  LIPA_CHECK_LAUNCH();
}
