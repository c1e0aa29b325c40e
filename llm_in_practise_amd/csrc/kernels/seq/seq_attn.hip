// Causal softmax attention over a slot-indexed K/V cache whose softmax weights are mixed across heads before they
// meet the values ("talking heads" after the softmax):  w'_h(i, j) = sum_g talk[h, g] w_g(i, j),
// o_h(i) = sum_j w'_h(i, j) v_kv(h)(j).
//
// Mixing is linear, so  o_h = sum_g talk[h, g] U[g, kv(h)]  with  U[g, c](i) = sum_j w_g(i, j) v_c(j): pass 1 is a
// flash-style single sweep per (query token, query head g) that accumulates its softmax weights against the values
// of ALL kv heads (G * dv columns) with a running maximum; keys may be cut into splits (decode: long caches, few
// rows).  Pass 2 merges the splits, normalises, mixes the heads with talk, applies the sigmoid output gate and writes
// the activation type.  Scores, weights and U are float.  One wave per (token, head, split): lanes own keys for
// q.k (each lane one key's full dot product, q broadcast from LDS), then own value columns for w.V.
#include "seq_common.h"

using namespace lipa;

constexpr int MAXC = 16;   // value columns per lane: G * dv <= 64 * MAXC

template <typename T>
__global__ __launch_bounds__(64) void k_talk_attn_partial(const T* __restrict__ q, int ldq, const T* __restrict__ kc,
                                                          const T* __restrict__ vc, float* __restrict__ pm,
                                                          float* __restrict__ pl, float* __restrict__ pu, int H, int G,
                                                          int dk, int dv, int max_len, int nsplit, float scale,
                                                          SeqDesc d) {
  extern __shared__ float sq[];
  const int t = blockIdx.x, g = blockIdx.y, z = blockIdx.z, lane = threadIdx.x;
  const int s = d.tok_seq[t], p = d.tok_pos[t], slot = d.slots[s];
  const int kh = g / (H / G), GV = G * dv;
  for (int i = lane; i < dk; i += 64) sq[i] = (float)q[(size_t)t * ldq + g * dk + i];
  __syncthreads();
  const int nkeys = p + 1, per = (nkeys + nsplit - 1) / nsplit;
  const int j0 = z * per, j1 = min(nkeys, j0 + per);
  const T* kbase = kc + ((size_t)slot * max_len) * (G * dk) + kh * dk;
  const T* vbase = vc + ((size_t)slot * max_len) * GV;
  float acc[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int jb = j0; jb < j1; jb += 64) {
    const int j = jb + lane;
    float sc = -INFINITY;
    if (j < j1) {
      const T* kr = kbase + (size_t)j * (G * dk);
      float a = 0.f;
      for (int i = 0; i < dk; ++i) a += sq[i] * (float)kr[i];
      sc = a * scale;
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float corr = expf(m - mn);          // m = -inf on the first chunk: exp(-inf) = 0
    const float w = j < j1 ? expf(sc - mn) : 0.f;
    l = l * corr + wave_sum(w);
    m = mn;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) acc[c] *= corr;
    const int cnt = min(64, j1 - jb);
    for (int jj = 0; jj < cnt; ++jj) {
      const float wj = __shfl(w, jj, 64);
      const T* vr = vbase + (size_t)(jb + jj) * GV;
#pragma unroll
      for (int c = 0; c < MAXC; ++c) {
        const int col = c * 64 + lane;
        if (col < GV) acc[c] += wj * (float)vr[col];
      }
    }
  }
  const size_t o = ((size_t)t * H + g) * nsplit + z;
  if (lane == 0) {
    pm[o] = m;
    pl[o] = l;
  }
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int col = c * 64 + lane;
    if (col < GV) pu[o * GV + col] = acc[c];
  }
}

// out[t, h, c] = sigmoid(gate[t, h*dv + c]) * sum_g talk[h, g] * U_g[kv(h)*dv + c] / l_g   (splits merged first)
template <typename T>
__global__ __launch_bounds__(64) void k_talk_attn_merge(const float* __restrict__ pm, const float* __restrict__ pl,
                                                        const float* __restrict__ pu, const float* __restrict__ talk,
                                                        const T* __restrict__ gate, int ldg, T* __restrict__ out, int H,
                                                        int G, int dv, int nsplit) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kh = h / (H / G), GV = G * dv;
  for (int c = lane; c < dv; c += 64) {
    float o = 0.f;
    for (int g = 0; g < H; ++g) {
      const size_t b = ((size_t)t * H + g) * nsplit;
      float mx = -INFINITY;
      for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, pm[b + z]);
      float l = 0.f, u = 0.f;
      for (int z = 0; z < nsplit; ++z) {
        const float e = expf(pm[b + z] - mx);
        l += e * pl[b + z];
        u += e * pu[(b + z) * GV + kh * dv + c];
      }
      o += talk[h * H + g] * (u / l);
    }
    out[(size_t)t * (H * dv) + h * dv + c] = (T)(o * sigmoidf_((float)gate[(size_t)t * ldg + h * dv + c]));
  }
}

int seq_attn_max_cols() { return 64 * MAXC; }

void seq_talk_attention(int code, const void* q, int ldq, const void* kc, const void* vc, float* pm, float* pl,
                        float* pu, const float* talk, const void* gate, int ldg, void* out, int H, int G, int dk, int dv,
                        int max_len, int nsplit, float scale, SeqDesc d, hipStream_t st) {
  if (d.Ttot == 0) return;
  SEQ_DISPATCH_T(code, {
    hipLaunchKernelGGL(k_talk_attn_partial<T>, dim3(d.Ttot, H, nsplit), dim3(64), sizeof(float) * dk, st, (const T*)q,
                       ldq, (const T*)kc, (const T*)vc, pm, pl, pu, H, G, dk, dv, max_len, nsplit, scale, d);
    hipLaunchKernelGGL(k_talk_attn_merge<T>, dim3(d.Ttot, H), dim3(64), 0, st, pm, pl, pu, talk, (const T*)gate, ldg,
                       (T*)out, H, G, dv, nsplit);
  });
  LIPA_CHECK_LAUNCH();
}
