// Attention whose scores are reshaped before the softmax, over the paged K/V pools:
//
//   s_g(i, j)  = softcap * tanh(scale * q_g(i) . k(j) / softcap)          (softcap 0: none)
//                - slope_g * (i - j)                                       (slopes null: none)
//   s'_h(i, j) = sum_g talk[h][g] * s_g(i, j)                              (talk null: identity)
//   visible j:   j <= i, same chunk of `chunk` positions (chunk 0: all), within `window` (0: all)
//   o_h(i)     = gate_h(i) * sum_j softmax_j(s'_h(i, .)) v(j)              (gate null: 1)
//
// The head mix couples all heads of a (query, key) pair, so one workgroup owns ONE query row with
// every head: per tile of 64 keys it forms the H x 64 raw scores, mixes them through LDS, runs one
// online-softmax step per head (a wave per head, a lane per key) and accumulates P.V with threads
// spread over (head, value channel).  Query rows are independent (row -> sequence, position), so a
// launch takes prompt portions and single decoded tokens alike.  K and V rows of key and value
// width Dk / Dv may differ.  Scores, softmax and the accumulators are fp32; q, K, V, gate logits
// and the output are the activation type (bf16 or fp32).
#include "common.h"

namespace la {

constexpr int AM_KT = 64;     // keys per tile = lanes of the softmax wave
constexpr int AM_NT = 256;
constexpr int AM_MAXO = 32;   // output accumulators per thread: H * Dv <= AM_NT * AM_MAXO

// q (fp32, LDS) . k (a cache row).  vec: the row is 16-byte aligned and D a multiple of the vector
template <typename AT>
LA_DEV float dot_row(const float* __restrict__ q, const AT* __restrict__ k, int D, bool vec);

template <>
LA_DEV float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int D, bool vec) {
  float a = 0.f;
  int d = 0;
  if (vec)
    for (; d + 4 <= D; d += 4) {
      const float4 kv = *(const float4*)(k + d);
      a = fmaf(q[d], kv.x, a); a = fmaf(q[d + 1], kv.y, a); a = fmaf(q[d + 2], kv.z, a); a = fmaf(q[d + 3], kv.w, a);
    }
  for (; d < D; ++d) a = fmaf(q[d], k[d], a);
  return a;
}
template <>
LA_DEV float dot_row<bf16>(const float* __restrict__ q, const bf16* __restrict__ k, int D, bool vec) {
  float a = 0.f;
  int d = 0;
  if (vec)
    for (; d + 8 <= D; d += 8) {
      const bf16x8 kv = *(const bf16x8*)(k + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) a = fmaf(q[d + e], (float)kv[e], a);
    }
  for (; d < D; ++d) a = fmaf(q[d], (float)k[d], a);
  return a;
}

template <typename AT>
__global__ __launch_bounds__(AM_NT) void attn_mix_rows_kernel(
    const AT* __restrict__ q, const AT* __restrict__ kc, const AT* __restrict__ vc, const int* __restrict__ row_seq,
    const int* __restrict__ pos, const int* __restrict__ bt, int maxb, int H, int G, int Dk, int Dv, int BS,
    float scale, float softcap, const float* __restrict__ slopes, const float* __restrict__ talk, int chunk,
    int window, const AT* __restrict__ gate, int ldg, AT* __restrict__ out) {
  extern __shared__ float lds[];
  float* qs = lds;                       // [H][Dk]
  float* s1 = qs + H * Dk;               // [H][KT] raw scores
  float* s2 = s1 + H * AM_KT;            // [H][KT] mixed scores, then probabilities
  float* mrun = s2 + H * AM_KT;          // [H] running max
  float* lrun = mrun + H;                // [H] running sum
  float* alpha = lrun + H;               // [H] rescale of this tile
  const int r = blockIdx.x, tid = threadIdx.x;
  const int i = pos[r];
  const int* tab = bt + (long)row_seq[r] * maxb;
  const int rep = H / G;
  const bool vec = (Dk * sizeof(AT)) % 16 == 0;
  for (int e = tid; e < H * Dk; e += AM_NT) qs[e] = (float)q[(long)r * H * Dk + e];
  for (int h = tid; h < H; h += AM_NT) { mrun[h] = -INFINITY; lrun[h] = 0.f; }
  int lo = 0;
  if (chunk > 0) lo = (i / chunk) * chunk;
  if (window > 0) lo = max(lo, i - window + 1);
  const int HV = H * Dv;
  float acc[AM_MAXO];
#pragma unroll
  for (int e = 0; e < AM_MAXO; ++e) acc[e] = 0.f;
  __syncthreads();
  for (int j0 = lo; j0 <= i; j0 += AM_KT) {
    const int nk = min(AM_KT, i + 1 - j0);
    // raw scores of every (head, key) pair of the tile
    for (int e = tid; e < H * AM_KT; e += AM_NT) {
      const int h = e / AM_KT, jj = e - h * AM_KT;
      float s = -INFINITY;
      if (jj < nk) {
        const int j = j0 + jj, blk = tab[j / BS], off = j % BS, g = h / rep;
        s = dot_row<AT>(qs + h * Dk, kc + (((long)blk * G + g) * BS + off) * Dk, Dk, vec) * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        if (slopes) s -= slopes[h] * (float)(i - j);
      }
      s1[e] = s;
    }
    __syncthreads();
    if (talk) {
      for (int e = tid; e < H * AM_KT; e += AM_NT) {
        const int h = e / AM_KT, jj = e - h * AM_KT;
        float m = -INFINITY;
        if (jj < nk) {
          m = 0.f;
          for (int g = 0; g < H; ++g) m = fmaf(talk[h * H + g], s1[g * AM_KT + jj], m);
        }
        s2[e] = m;
      }
    } else {
      for (int e = tid; e < H * AM_KT; e += AM_NT) s2[e] = s1[e];
    }
    __syncthreads();
    // one online-softmax step per head: a wave per head, a lane per key
    for (int h = tid >> 6; h < H; h += AM_NT / 64) {
      const int lane = tid & 63;
      const float s = s2[h * AM_KT + lane];
      const float mo = mrun[h];
      const float mn = fmaxf(mo, wave_max(s));
      const float p = (s == -INFINITY) ? 0.f : __expf(s - mn);
      const float ps = wave_sum(p);
      s2[h * AM_KT + lane] = p;
      if (lane == 0) {
        const float a = (mo == -INFINITY) ? 0.f : __expf(mo - mn);
        alpha[h] = a;
        lrun[h] = lrun[h] * a + ps;
        mrun[h] = mn;
      }
    }
    __syncthreads();
    // o[h][d] = o[h][d] * alpha[h] + sum_jj p[h][jj] * V[j][g(h)][d]
#pragma unroll
    for (int e = 0; e < AM_MAXO; ++e) {
      const int o = tid + e * AM_NT;
      if (o < HV) {
        const int h = o / Dv, d = o - h * Dv, g = h / rep;
        float a = acc[e] * alpha[h];
        for (int jj = 0; jj < nk; ++jj) {
          const int j = j0 + jj, blk = tab[j / BS], off = j % BS;
          a = fmaf(s2[h * AM_KT + jj], (float)vc[(((long)blk * G + g) * BS + off) * Dv + d], a);
        }
        acc[e] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < AM_MAXO; ++e) {
    const int o = tid + e * AM_NT;
    if (o < HV) {
      const int h = o / Dv;
      float v = acc[e] / lrun[h];
      if (gate) v *= 1.f / (1.f + __expf(-(float)gate[(long)r * ldg + h]));
      out[(long)r * HV + o] = (AT)v;
    }
  }
}

}  // namespace la

extern "C" int la_attn_mix_rows(int f32, const void* q, const void* kc, const void* vc, const void* row_seq,
                                const void* pos, const void* bt, int maxb, int T, int H, int G, int Dk, int Dv, int BS,
                                float scale, float softcap, const void* slopes, const void* talk, int chunk, int window,
                                const void* gate, int ldg, void* out, void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || H * Dv > AM_NT * AM_MAXO) return -1;
  const size_t shm = sizeof(float) * ((size_t)H * Dk + 2 * (size_t)H * AM_KT + 3 * (size_t)H);
  if (shm > 160 * 1024) return -2;
  hipStream_t s = (hipStream_t)stream;
  if (f32) {
    if (shm > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_mix_rows_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
    hipLaunchKernelGGL((attn_mix_rows_kernel<float>), dim3(T), dim3(AM_NT), shm, s, (const float*)q, (const float*)kc,
                       (const float*)vc, (const int*)row_seq, (const int*)pos, (const int*)bt, maxb, H, G, Dk, Dv, BS,
                       scale, softcap, (const float*)slopes, (const float*)talk, chunk, window, (const float*)gate, ldg,
                       (float*)out);
  } else {
    if (shm > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_mix_rows_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
    hipLaunchKernelGGL((attn_mix_rows_kernel<bf16>), dim3(T), dim3(AM_NT), shm, s, (const bf16*)q, (const bf16*)kc,
                       (const bf16*)vc, (const int*)row_seq, (const int*)pos, (const int*)bt, maxb, H, G, Dk, Dv, BS,
                       scale, softcap, (const float*)slopes, (const float*)talk, chunk, window, (const bf16*)gate, ldg,
                       (bf16*)out);
  }
  return (int)hipGetLastError();
}
