// Short causal convolution over time on projected q | k | v channels, with the paged K/V append
// and the cross-layer value mix fused in, plus the per-sequence tail state that lets a sequence
// continue in a later step (prompt portions, decoding).
//
//   y[t][c] = sum_{j < taps} w[c][j] * u[t - (taps - 1) + j][c]        (zeros before position 0)
//
// u is the projection output [T, ldp] (q channels, then k, then v); rows of one sequence portion are
// consecutive.  Tokens before the portion come from the sequence's state slot, which holds the last
// taps - 1 projected rows; what lies before position 0 reads as zero whatever the slot holds, so a
// slot needs no clearing when another sequence takes it over.
//
// Outputs: q rows [T, Cq]; k into the paged K pool [blocks, G, BS, Dk]; v -- optionally mixed with
// the first mixing layer's values, v <- (1 - lam) v + lam v_first -- into the V pool, which is
// transposed per 8 keys, [blocks, G, BS / 8, Dv, 8] (the P.V matrix instruction's operand layout).
// Accumulation, the mix and lam are fp32; storage is the activation type.
#include "common.h"

namespace la {

template <typename AT>
LA_DEV float ld(const AT* p) { return (float)*p; }

template <typename AT, bool SINGLE>
__global__ __launch_bounds__(256) void shortconv_kv_kernel(
    const AT* __restrict__ u, int ldp, const float* __restrict__ w, int taps, int Cq, int Ck, int Cv,
    const int* __restrict__ row_seq, const int* __restrict__ cu_q, const int* __restrict__ pos,
    const int* __restrict__ slots, const int* __restrict__ sslot, AT* __restrict__ state,
    AT* __restrict__ q_out, AT* __restrict__ kc, AT* __restrict__ vc, int G, int Dk, int Dv, int BS,
    const float* __restrict__ vfirst_in, float* __restrict__ vfirst_out, const float* __restrict__ lam_p) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int C = Cq + Ck + Cv;
  if (c >= C) return;
  const int seq = row_seq[r];
  const int c0 = cu_q[seq];
  const int m = r - c0;          // rows of this portion before r
  const int p = pos[r];
  const int ss = sslot[seq];
  const long st_base = (long)ss * (taps - 1) * C;
  float acc = 0.f;
  float hist[8];                 // SINGLE: the tail read from the state (taps - 1 <= 8)
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j;  // tokens back
    float x = 0.f;
    if (d <= p) {                // position p - d exists
      if (d <= m) {
        x = ld(u + (long)(r - d) * ldp + c);
      } else if (ss >= 0) {
        x = ld(state + st_base + (long)(taps - 1 - (d - m)) * C + c);
      }
    }
    if (SINGLE && d > 0) hist[taps - 1 - d] = x;
    acc = fmaf(w[(long)c * taps + j], x, acc);
  }
  if (SINGLE && ss >= 0 && taps > 1) {
    // one row per sequence: this thread is the only reader and writer of (slot, channel)
    for (int i = 0; i + 1 < taps - 1; ++i) state[st_base + (long)i * C + c] = (AT)hist[i + 1];
    state[st_base + (long)(taps - 2) * C + c] = u[(long)r * ldp + c];
  }
  const int slot = slots[r];
  if (c < Cq) {
    q_out[(long)r * Cq + c] = (AT)acc;
  } else if (c < Cq + Ck) {
    if (slot >= 0) {
      const int ck = c - Cq, g = ck / Dk, d = ck - g * Dk;
      const int blk = slot / BS, off = slot - blk * BS;
      kc[(((long)blk * G + g) * BS + off) * Dk + d] = (AT)acc;
    }
  } else {
    const int cv = c - Cq - Ck;
    float v = acc;
    if (vfirst_out) vfirst_out[(long)r * Cv + cv] = v;
    if (vfirst_in) {
      const float lam = *lam_p;
      v = (1.f - lam) * v + lam * vfirst_in[(long)r * Cv + cv];
    }
    if (slot >= 0) {
      const int g = cv / Dv, d = cv - g * Dv;
      const int blk = slot / BS, off = slot - blk * BS;
      vc[((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7)] = (AT)v;
    }
  }
}

// bf16 with every width a multiple of 8: one thread per 8 consecutive channels, 16-byte loads of
// the projection rows and the state, 16-byte stores of q, k and the state (v stays element-wise:
// its pages are transposed per 8 keys).  Same arithmetic as shortconv_kv_kernel; the weights come
// tap-major, wt [taps, C], so a thread's 8 weights of one tap are two 16-byte loads.
template <bool SINGLE>
__global__ __launch_bounds__(256) void shortconv_kv8_kernel(
    const bf16* __restrict__ u, int ldp, const float* __restrict__ wt, int taps, int Cq, int Ck, int Cv,
    const int* __restrict__ row_seq, const int* __restrict__ cu_q, const int* __restrict__ pos,
    const int* __restrict__ slots, const int* __restrict__ sslot, bf16* __restrict__ state,
    bf16* __restrict__ q_out, bf16* __restrict__ kc, bf16* __restrict__ vc, int G, int Dk, int Dv, int BS,
    const float* __restrict__ vfirst_in, float* __restrict__ vfirst_out, const float* __restrict__ lam_p) {
  const int r = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
  const int C = Cq + Ck + Cv;
  if (c >= C) return;
  const int seq = row_seq[r];
  const int m = r - cu_q[seq];
  const int p = pos[r];
  const int ss = sslot[seq];
  bf16* st = state + (long)ss * (taps - 1) * C + c;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j;
    bf16x8 x = {};
    if (d <= p) {
      if (d <= m) x = *(const bf16x8*)(u + (long)(r - d) * ldp + c);
      else if (ss >= 0) x = *(const bf16x8*)(st + (long)(taps - 1 - (d - m)) * C);
    }
    if (SINGLE && ss >= 0 && j >= 1) *(bf16x8*)(st + (long)(j - 1) * C) = x;   // row j - 1 <- old row j (or u for the last)
    const float4 w0 = *(const float4*)(wt + (long)j * C + c), w1 = *(const float4*)(wt + (long)j * C + c + 4);
    acc[0] = fmaf(w0.x, (float)x[0], acc[0]); acc[1] = fmaf(w0.y, (float)x[1], acc[1]);
    acc[2] = fmaf(w0.z, (float)x[2], acc[2]); acc[3] = fmaf(w0.w, (float)x[3], acc[3]);
    acc[4] = fmaf(w1.x, (float)x[4], acc[4]); acc[5] = fmaf(w1.y, (float)x[5], acc[5]);
    acc[6] = fmaf(w1.z, (float)x[6], acc[6]); acc[7] = fmaf(w1.w, (float)x[7], acc[7]);
  }
  const int slot = slots[r];
  if (c < Cq) {
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)acc[e];
    *(bf16x8*)(q_out + (long)r * Cq + c) = o;
  } else if (c < Cq + Ck) {
    if (slot >= 0) {
      const int ck = c - Cq, g = ck / Dk, d = ck - g * Dk;
      const int blk = slot / BS, off = slot - blk * BS;
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (bf16)acc[e];
      *(bf16x8*)(kc + (((long)blk * G + g) * BS + off) * Dk + d) = o;
    }
  } else {
    const int cv = c - Cq - Ck;
    if (vfirst_out) {
      *(float4*)(vfirst_out + (long)r * Cv + cv) = float4{acc[0], acc[1], acc[2], acc[3]};
      *(float4*)(vfirst_out + (long)r * Cv + cv + 4) = float4{acc[4], acc[5], acc[6], acc[7]};
    }
    if (vfirst_in) {
      const float lam = *lam_p;
      const float4 a = *(const float4*)(vfirst_in + (long)r * Cv + cv), b = *(const float4*)(vfirst_in + (long)r * Cv + cv + 4);
      const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = (1.f - lam) * acc[e] + lam * f[e];
    }
    if (slot >= 0) {
      const int g = cv / Dv, d = cv - g * Dv;
      const int blk = slot / BS, off = slot - blk * BS;
      bf16* vp = vc + ((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7);
#pragma unroll
      for (int e = 0; e < 8; ++e) vp[e * 8] = (bf16)acc[e];
    }
  }
}

// New tail of every sequence of the batch: the last taps - 1 projected rows up to the end of its
// portion.  Rows the portion does not cover shift down from the old tail (ascending order: each
// read is of a higher index than any write before it).
template <typename AT>
__global__ __launch_bounds__(256) void shortconv_state_kernel(const AT* __restrict__ u, int ldp, int taps, int C,
                                                              const int* __restrict__ cu_q,
                                                              const int* __restrict__ sslot, AT* __restrict__ state) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int ss = sslot[seq];
  if (ss < 0) return;
  const int c0 = cu_q[seq], n = cu_q[seq + 1] - c0;
  AT* st = state + (long)ss * (taps - 1) * C + c;
  for (int i = 0; i < taps - 1; ++i) {
    const int src = n - (taps - 1) + i;   // row of the portion, or before it
    st[(long)i * C] = src >= 0 ? u[(long)(c0 + src) * ldp + c] : st[(long)(i + n) * C];
  }
}

}  // namespace la

// f32: 1 = fp32 activations / cache / state, 0 = bf16.  single: every sequence brings exactly one
// row (decode batches): the state update is fused into the convolution launch.
// wt: the weights once more, tap-major [taps, C] (may be null: then the scalar kernel runs)
extern "C" int la_shortconv_kv(int f32, int single, const void* u, int ldp, const void* w, const void* wt, int taps, int Cq, int Ck,
                               int Cv, const void* row_seq, const void* cu_q, const void* pos, const void* slots,
                               const void* sslot, void* state, void* q_out, void* kc, void* vc, int G, int Dk,
                               int Dv, int BS, const void* vfirst_in, void* vfirst_out, const void* lam, int T,
                               int nseq, void* stream) {
  using namespace la;
  const int C = Cq + Ck + Cv;
  if (taps < 1 || taps > 9 || T <= 0 || C <= 0 || Ck != G * Dk || Cv != G * Dv || (single && nseq != T) || (BS & 7)) return -1;
  dim3 grid((C + 255) / 256, T), gs((C + 255) / 256, nseq);
  hipStream_t s = (hipStream_t)stream;
#define LA_SC(AT, SG)                                                                                          \
  hipLaunchKernelGGL((shortconv_kv_kernel<AT, SG>), grid, dim3(256), 0, s, (const AT*)u, ldp, (const float*)w, \
                     taps, Cq, Ck, Cv, (const int*)row_seq, (const int*)cu_q, (const int*)pos,                \
                     (const int*)slots, (const int*)sslot, (AT*)state, (AT*)q_out, (AT*)kc, (AT*)vc, G, Dk,   \
                     Dv, BS, (const float*)vfirst_in, (float*)vfirst_out, (const float*)lam)
  const bool vec8 = !f32 && wt && !((uintptr_t)wt & 15) && !(Cq & 7) && !(Dk & 7) && !(Dv & 7) && !(ldp & 7) && !((uintptr_t)u & 15) &&
                    !((uintptr_t)state & 15) && !((uintptr_t)kc & 15) && !((uintptr_t)vfirst_in & 15) &&
                    !((uintptr_t)vfirst_out & 15);
  if (vec8) {
    dim3 g8((C / 8 + 255) / 256, T);
#define LA_SC8(SG)                                                                                              \
  hipLaunchKernelGGL((shortconv_kv8_kernel<SG>), g8, dim3(256), 0, s, (const bf16*)u, ldp, (const float*)wt, taps, \
                     Cq, Ck, Cv, (const int*)row_seq, (const int*)cu_q, (const int*)pos, (const int*)slots,      \
                     (const int*)sslot, (bf16*)state, (bf16*)q_out, (bf16*)kc, (bf16*)vc, G, Dk, Dv, BS,         \
                     (const float*)vfirst_in, (float*)vfirst_out, (const float*)lam)
    if (single) LA_SC8(true); else LA_SC8(false);
#undef LA_SC8
  } else if (f32) {
    if (single) LA_SC(float, true); else LA_SC(float, false);
  } else {
    if (single) LA_SC(bf16, true); else LA_SC(bf16, false);
  }
#undef LA_SC
  if (!single && taps > 1) {
    if (f32)
      hipLaunchKernelGGL((shortconv_state_kernel<float>), gs, dim3(256), 0, s, (const float*)u, ldp, taps, C,
                         (const int*)cu_q, (const int*)sslot, (float*)state);
    else
      hipLaunchKernelGGL((shortconv_state_kernel<bf16>), gs, dim3(256), 0, s, (const bf16*)u, ldp, taps, C,
                         (const int*)cu_q, (const int*)sslot, (bf16*)state);
  }
  return (int)hipGetLastError();
}
