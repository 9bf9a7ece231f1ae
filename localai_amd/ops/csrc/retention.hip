// Retention: linear attention with a fixed decay per head, no softmax and no denominator.
//
//   q_t, k_t rotated on their first `rot` dims (pair (i, i + rot / 2), angle pos * freq[i], fp32),
//   k_t times Dk^-1/2;   S_t = decay_h S_(t-1) + k_t v_t^T   (Dk x Dv, fp32);   o_t = S_t^T q_t
//   out_t = o_t / sqrt(mean_d o_t[d]^2 + eps) * silu(gate_t)          (mean over the head's Dv)
//
// The state of a sequence lives in a slot pool [slots][H][Dv][Dk] (value-column major) between
// launches: a portion starting at position 0 starts from zeros whatever the slot holds, any other
// portion from the slot, and every portion leaves its end state there.
//
// retention_rot_kernel: rotated q and scaled rotated k of every row, once, as fp32 [T][2][H][Dk].
// retention_scan_kernel: workgroup = (sequence portion, head, slice of value columns).  A column's
// Dk state entries sit in the registers of P lanes (R each, rows interleaved over the lanes, so LDS
// and state accesses of a lane group are consecutive); tokens are staged through LDS in chunks
// (q, k, v) and scanned in order, o_t[c] reduced over the P lanes by shuffles.  P grows (narrower
// column slices, more workgroups) until a launch has about four workgroups per compute unit: a scan
// is a chain of dependent steps, so it is the number of resident waves that hides its latencies.  A
// decode batch is the same launch with one-token portions: it then streams each state once, which is
// its memory bound.  retention_out_kernel: the per-head unit norm and the gate.
#include "common.h"

namespace la {

constexpr int RT_NT = 256;
constexpr int RT_TC = 16;     // tokens staged per chunk

// qk[t][0][h][d] = rotated q, qk[t][1][h][d] = rotated k * kscale (fp32): a thread per (row, head, pair or plain dim)
template <typename AT>
__global__ __launch_bounds__(256) void retention_rot_kernel(const AT* __restrict__ src, int ld, int H, int Dk,
                                                            const int* __restrict__ pos, const float* __restrict__ freqs,
                                                            float mag, int rot, float kscale, float* __restrict__ qk,
                                                            long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int half = rot >> 1, per = Dk - half;        // units per head: rot / 2 pairs, then Dk - rot plain dims
  const long th = e / per;
  const int u = (int)(e - th * per);
  const long t = th / H;
  const int h = (int)(th - t * H);
  const AT* q = src + t * ld + (long)h * Dk;
  const AT* k = q + (long)H * Dk;
  float* qo = qk + (t * 2 * H + h) * Dk;
  float* ko = qo + (long)H * Dk;
  if (u < half) {
    const float ang = (float)pos[t] * freqs[u];
    const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
    const float qu = (float)q[u], qw = (float)q[u + half], ku = (float)k[u], kw = (float)k[u + half];
    qo[u] = qu * cs - qw * sn;
    qo[u + half] = qw * cs + qu * sn;
    ko[u] = (ku * cs - kw * sn) * kscale;
    ko[u + half] = (kw * cs + ku * sn) * kscale;
  } else {
    const int d = u + half;
    qo[d] = (float)q[d];
    ko[d] = (float)k[d] * kscale;
  }
}

template <typename AT, int R>
__global__ __launch_bounds__(RT_NT) void retention_scan_kernel(
    const AT* __restrict__ src, int ld, const float* __restrict__ qk, int H, int Dk, int Dv, const int* __restrict__ pos,
    const int* __restrict__ cu_q, const int* __restrict__ sslots, float* __restrict__ state,
    const float* __restrict__ decay, float* __restrict__ o, int P) {
  extern __shared__ float lds[];
  const int DkP = P * R;                 // padded key width (rows beyond Dk hold zeros)
  const int cpw = RT_NT / P;             // value columns of this workgroup
  float* qs = lds;                       // [TC][DkP]
  float* ks = qs + RT_TC * DkP;          // [TC][DkP]
  float* vs = ks + RT_TC * DkP;          // [TC][cpw]
  const int seq = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * cpw;
  const int tid = threadIdx.x, part = tid % P, cl = tid / P, c = c0 + cl;
  const int a = cu_q[seq], b = cu_q[seq + 1];
  if (b <= a) return;
  const int slot = sslots[seq];
  const float dec = decay[h];
  float S[R];
  float* st = (slot >= 0 && c < Dv) ? state + (((long)slot * H + h) * Dv + c) * Dk : nullptr;
  const bool fresh = pos[a] == 0;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int r = j * P + part;
    S[j] = (st && !fresh && r < Dk) ? st[r] : 0.f;
  }
  const long vcol = 2L * H * Dk + (long)h * Dv;
  for (int t0 = a; t0 < b; t0 += RT_TC) {
    const int n = min(RT_TC, b - t0);
    __syncthreads();
    for (int e = tid; e < n * DkP; e += RT_NT) {
      const int tt = e / DkP, d = e - tt * DkP;
      float qv = 0.f, kv = 0.f;
      if (d < Dk) {
        const float* row = qk + ((long)(t0 + tt) * 2 * H + h) * Dk + d;
        qv = row[0];
        kv = row[(long)H * Dk];
      }
      qs[e] = qv;
      ks[e] = kv;
    }
    for (int e = tid; e < n * cpw; e += RT_NT) {
      const int tt = e / cpw, cc = e - tt * cpw;
      vs[e] = (c0 + cc < Dv) ? (float)src[(long)(t0 + tt) * ld + vcol + c0 + cc] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float vv = vs[tt * cpw + cl];
      const float* kr = ks + tt * DkP + part;
      const float* qr = qs + tt * DkP + part;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        S[j] = fmaf(dec, S[j], kr[j * P] * vv);
        acc = fmaf(S[j], qr[j * P], acc);
      }
      for (int w = P >> 1; w > 0; w >>= 1) acc += __shfl_xor(acc, w, 64);
      if (part == 0 && c < Dv) o[(long)(t0 + tt) * H * Dv + (long)h * Dv + c] = acc;
    }
  }
  if (st) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int r = j * P + part;
      if (r < Dk) st[r] = S[j];
    }
  }
}

// out[t][h][:] = o / sqrt(mean(o^2) + eps) * silu(gate): a wave per (token, head)
template <typename AT>
__global__ __launch_bounds__(256) void retention_out_kernel(const float* __restrict__ o, const AT* __restrict__ src, int ld,
                                                            long gcol, int H, int Dv, long rows, float eps,
                                                            AT* __restrict__ out) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const long t = r / H;
  const int h = (int)(r - t * H);
  const float* orow = o + r * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) ss = fmaf(orow[d], orow[d], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
  const AT* g = src + t * ld + gcol + (long)h * Dv;
  for (int d = lane; d < Dv; d += 64) {
    const float gv = (float)g[d];
    out[r * Dv + d] = (AT)(orow[d] * inv * (gv / (1.f + expf(-gv))));
  }
}

template <typename AT>
static int launch_scan(const AT* src, int ld, int T, int nseq, int H, int Dk, int Dv, const int* pos, const int* cu_q,
                       const int* sslots, float* state, const float* decay, const float* freqs, float mag, int rot,
                       float* qk, float* o, hipStream_t st) {
  const float kscale = 1.f / sqrtf((float)Dk);
  {
    const long total = (long)T * H * (Dk - (rot >> 1));
    hipLaunchKernelGGL(retention_rot_kernel<AT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, src, ld, H, Dk, pos,
                       freqs, mag, rot, kscale, qk, total);
  }
  // P lanes per value column (power of two), R rows per lane: P * R >= Dk with R <= 32; more lanes per
  // column while the launch has fewer than about four workgroups per compute unit
  int P = 8;
  while (P < 64 && (Dk + P - 1) / P > 32) P <<= 1;
  if ((Dk + P - 1) / P > 32) return -5;
  while (P < 64 && (Dk + P - 1) / P > 2 && (long)nseq * H * ((Dv + RT_NT / P - 1) / (RT_NT / P)) < 1024) P <<= 1;
  const int need = (Dk + P - 1) / P;
  const int cpw = RT_NT / P;
  dim3 grid(nseq, H, (Dv + cpw - 1) / cpw);
#define LA_RT_LAUNCH(RR)                                                                                              \
  {                                                                                                                   \
    const size_t shm = (size_t)(2 * RT_TC * P * RR + RT_TC * cpw) * sizeof(float);                                    \
    if (shm > 150 * 1024) return -6;                                                                                  \
    if (shm > 48 * 1024)                                                                                              \
      (void)hipFuncSetAttribute((const void*)retention_scan_kernel<AT, RR>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)shm);                                                                            \
    hipLaunchKernelGGL((retention_scan_kernel<AT, RR>), grid, dim3(RT_NT), shm, st, src, ld, (const float*)qk, H, Dk, \
                       Dv, pos, cu_q, sslots, state, decay, o, P);                                                    \
  }
  if (need <= 1) LA_RT_LAUNCH(1)
  else if (need <= 2) LA_RT_LAUNCH(2)
  else if (need <= 4) LA_RT_LAUNCH(4)
  else if (need <= 8) LA_RT_LAUNCH(8)
  else if (need <= 16) LA_RT_LAUNCH(16)
  else LA_RT_LAUNCH(32)
#undef LA_RT_LAUNCH
  return (int)hipGetLastError();
}

}  // namespace la

extern "C" int la_retention(int f32, const void* src, int T, int nseq, int H, int Dk, int Dv, const void* pos,
                            const void* cu_q, const void* sslots, void* state, int nslots, const void* decay,
                            const void* freqs, float mag, int rot, float eps, void* qk, void* o, void* out, void* stream) {
  using namespace la;
  if (T <= 0 || nseq <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || (rot & 1) || rot > Dk || nslots <= 0) return -1;
  if (!src || !pos || !cu_q || !sslots || !state || !decay || !freqs || !qk || !o || !out) return -2;
  hipStream_t st = (hipStream_t)stream;
  const int ld = 2 * H * Dk + 2 * H * Dv;
  const long gcol = 2L * H * Dk + (long)H * Dv, rows = (long)T * H;
  int rc;
  if (f32) {
    rc = launch_scan<float>((const float*)src, ld, T, nseq, H, Dk, Dv, (const int*)pos, (const int*)cu_q,
                            (const int*)sslots, (float*)state, (const float*)decay, (const float*)freqs, mag, rot,
                            (float*)qk, (float*)o, st);
    if (rc) return rc;
    hipLaunchKernelGGL(retention_out_kernel<float>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o,
                       (const float*)src, ld, gcol, H, Dv, rows, eps, (float*)out);
  } else {
    rc = launch_scan<bf16>((const bf16*)src, ld, T, nseq, H, Dk, Dv, (const int*)pos, (const int*)cu_q,
                           (const int*)sslots, (float*)state, (const float*)decay, (const float*)freqs, mag, rot,
                           (float*)qk, (float*)o, st);
    if (rc) return rc;
    hipLaunchKernelGGL(retention_out_kernel<bf16>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o,
                       (const bf16*)src, ld, gcol, H, Dv, rows, eps, (bf16*)out);
  }
  return (int)hipGetLastError();
}
