// Attention over a latent cache on the matrix cores (bf16): every query head of a token reads the
// SAME cached row per key -- one kv head whose row [c (Dv) | rotated part] is the key, and whose
// first Dv columns are also the value.  So the heads of a token are the 16 rows of an MFMA tile and
// a key tile is shared by all of them:
//
//   workgroup = (query token, block of 16 heads[, key split]), 4 waves, per tile of 32 keys:
//     1. the 32 cached rows -> LDS (16-byte loads through the block table, issued a tile ahead into
//        registers), once for QK^T and PV
//     2. S = Q K^T: MFMA 16x16x32 bf16, wave (kb, kh) = keys 16 kb.., half kh of the key width; Q
//        fragments stay in registers over the key loop; partial sums of the two halves -> LDS
//     3. online softmax in fp32: 16 lanes a row, two keys a lane; probabilities -> LDS as bf16 in
//        A-operand layout, the rescale factor of the tile per row
//     4. O += P V: wave w owns the groups of 32 value columns w, w + 4, ...; B fragments (8 keys of
//        one column per lane) are gathered from the row-major LDS tile, which saves a transposed copy
//        -- as dwords, two columns at once, the even and the odd columns of a group as two MFMAs
//   epilogue: 1 / l, sigmoid head gate; with key splits the unnormalised (m, l, o) per split, merged
//   by latent_merge_kernel.
//
// A launch takes prompt portions and decoded tokens alike (row -> sequence, position).  Visible keys:
// j <= i, and i - j < window when window > 0.
#include "common.h"

namespace la {

constexpr int AL_KT = 32;        // keys per tile
constexpr int AL_QF = 10;        // Q fragments a wave keeps: half of Dk / 32 <= 10  (Dk <= 640)
constexpr int AL_NB = 8;         // value column blocks a wave owns: Dv / 16 / 4 <= 8  (Dv <= 512)
constexpr int AL_PRE = (AL_KT * (64 * AL_QF / 8) + 255) / 256;   // 16-byte chunks of a key tile per thread
constexpr int AL_SS = AL_KT + 1; // fp32 score row stride
constexpr int AL_PS = AL_KT + 8; // bf16 probability row stride (16-byte aligned rows)

__global__ __launch_bounds__(256) void attn_latent_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const int* __restrict__ row_seq, const int* __restrict__ pos,
    const int* __restrict__ bt, int maxb, int H, int Dk, int Dv, int BS, float scale, int window,
    const bf16* __restrict__ gate, int ldg, bf16* __restrict__ out, int nsplit, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  extern __shared__ float lds[];
  const int KS = Dk + 8;                       // LDS row stride of the key tile (bf16), rows 16-byte aligned
  float* sp = lds;                             // [2][16][AL_SS] partial scores of the two key-width halves
  float* alpha = sp + 2 * 16 * AL_SS;          // [16]
  float* lfin = alpha + 16;                    // [16]
  float* mfin = lfin + 16;                     // [16]
  bf16* pb = (bf16*)(mfin + 16);               // [16][AL_PS]
  bf16* ks = pb + 16 * AL_PS;                  // [AL_KT][KS]
  const int r = blockIdx.x, h0 = blockIdx.y * 16, split = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fr = lane & 15, fq = lane >> 4;
  const int nh = min(16, H - h0);
  const int i = pos[r];
  const int* tab = bt + (long)row_seq[r] * maxb;
  const int KC = Dk >> 5, KH = (KC + 1) >> 1;  // k-steps, k-steps of the first half
  const int kb = wave & 1, kh = wave >> 1;
  const int ks0 = kh * KH, nks = kh ? KC - KH : KH;
  // Q fragments (A operand: row fr = head, k = 32 step + 8 fq)
  bf16x8 qa[AL_QF];
  {
    const bf16* qp = q + ((long)r * H + h0 + min(fr, nh - 1)) * Dk;
#pragma unroll
    for (int s = 0; s < AL_QF; ++s) {
      bf16x8 v = {};
      if (s < nks) v = *(const bf16x8*)(qp + 32 * (ks0 + s) + 8 * fq);
      qa[s] = v;
    }
  }
  f32x4 o[AL_NB];
#pragma unroll
  for (int b = 0; b < AL_NB; ++b) o[b] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int NGT = Dv >> 5;                     // groups of 32 value columns in all
  // softmax bookkeeping: thread (row srow, lanes 16) keeps the row's running max / sum in registers
  const int srow = tid >> 4, sc = tid & 15;
  float mrun = -INFINITY, lrun = 0.f;
  const int lo = window > 0 ? max(0, i - window + 1) : 0;
  const int cpr = Dk >> 3;                     // 16-byte chunks per cached row
  // a tile's cached rows travel global -> registers -> LDS; the loads of the NEXT tile are issued
  // before this tile's arithmetic, so their latency hides behind it (rows past the query are zero)
  bf16x8 pre[AL_PRE];
  int pkk[AL_PRE];                             // chunk u of this thread: tile row, or -1
#pragma unroll
  for (int u = 0; u < AL_PRE; ++u) {
    const int c = tid + 256 * u;
    pkk[u] = c < AL_KT * cpr ? c / cpr : -1;
  }
  const int bs_shift = (BS & (BS - 1)) == 0 ? __builtin_ctz(BS) : -1;
  auto fetch = [&](int j0) {
#pragma unroll
    for (int u = 0; u < AL_PRE; ++u) {
      bf16x8 v = {};
      const int kk = pkk[u], j = j0 + kk;
      if (kk >= 0 && j <= i) {
        const int blk = bs_shift >= 0 ? j >> bs_shift : j / BS;
        const long slot = (long)tab[blk] * BS + (j - blk * BS);
        v = *(const bf16x8*)(kc + slot * Dk + 8 * (tid + 256 * u - kk * cpr));
      }
      pre[u] = v;
    }
  };
  const int jfirst = (lo / AL_KT + split) * AL_KT;
  if (jfirst <= i) fetch(jfirst);
  for (int j0 = jfirst; j0 <= i; j0 += AL_KT * nsplit) {
    __syncthreads();                           // the previous tile's PV has read ks / pb / alpha
    // ---- 1: key tile -> LDS
#pragma unroll
    for (int u = 0; u < AL_PRE; ++u) {
      const int kk = pkk[u];
      if (kk >= 0) *(bf16x8*)(ks + kk * KS + 8 * (tid + 256 * u - kk * cpr)) = pre[u];
    }
    if (j0 + AL_KT * nsplit <= i) fetch(j0 + AL_KT * nsplit);
    __syncthreads();
    // ---- 2: partial scores of this wave's 16 keys over its half of the key width
    {
      f32x4 a = {0.f, 0.f, 0.f, 0.f};
      const bf16* kp = ks + (16 * kb + fr) * KS + 32 * ks0 + 8 * fq;
#pragma unroll
      for (int s = 0; s < AL_QF; ++s)
        if (s < nks) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[s], *(const bf16x8*)(kp + 32 * s), a, 0, 0, 0);
#pragma unroll
      for (int e = 0; e < 4; ++e) sp[(kh * 16 + 4 * fq + e) * AL_SS + 16 * kb + fr] = a[e];
    }
    __syncthreads();
    // ---- 3: online softmax, row srow, keys sc and sc + 16
    {
      float s[2], p[2];
      float mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int kk = sc + 16 * e, j = j0 + kk;
        s[e] = (j <= i && j >= lo) ? (sp[srow * AL_SS + kk] + sp[(16 + srow) * AL_SS + kk]) * scale : -INFINITY;
        mx = fmaxf(mx, s[e]);
      }
      mx = group_max<16>(mx);
      const float mn = fmaxf(mrun, mx);
      float sum = 0.f;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        p[e] = s[e] == -INFINITY ? 0.f : __expf(s[e] - mn);
        sum += p[e];
        pb[srow * AL_PS + sc + 16 * e] = (bf16)p[e];
      }
      sum = group_sum<16>(sum);
      const float a = mrun == -INFINITY ? 0.f : __expf(mrun - mn);
      lrun = lrun * a + sum;
      mrun = mn;
      if (sc == 0) alpha[srow] = a;
    }
    __syncthreads();
    // ---- 4: O = O * alpha + P V over this wave's value column blocks
    {
      const bf16x8 pa = *(const bf16x8*)(pb + fr * AL_PS + 8 * fq);
      float al[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) al[e] = alpha[4 * fq + e];
      // value columns in groups of 32: group m = wave + 4 bp.  A lane gathers DWORDS -- columns 32 m +
      // 2 fr and + 1 of its 8 keys -- whose low halves are the B fragment of accumulator 2 bp (the even
      // columns of the group) and whose high halves that of 2 bp + 1 (the odd ones): half the gathers
#pragma unroll
      for (int bp = 0; bp < AL_NB / 2; ++bp) {
        const int m = wave + 4 * bp;
        if (m < NGT) {
          const uint32_t* vp = (const uint32_t*)(ks + (8 * fq) * KS + 32 * m) + fr;
          uint32_t d[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) d[e] = vp[e * (KS >> 1)];
          u32x4 ev, od;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            ev[k] = (d[2 * k] & 0xffffu) | (d[2 * k + 1] << 16);
            od[k] = (d[2 * k] >> 16) | (d[2 * k + 1] & 0xffff0000u);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) { o[2 * bp][e] *= al[e]; o[2 * bp + 1][e] *= al[e]; }
          o[2 * bp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8, ev), o[2 * bp], 0, 0, 0);
          o[2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8, od), o[2 * bp + 1], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();
  if (sc == 0) { lfin[srow] = lrun; mfin[srow] = mrun; }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int hr = 4 * fq + e;
    if (hr >= nh) continue;
    const int h = h0 + hr;
    if (nsplit > 1) {
      const long base = ((long)r * H + h) * nsplit + split;
      if (fr == 0 && wave == 0) { part_ml[2 * base] = mfin[hr]; part_ml[2 * base + 1] = lfin[hr]; }
#pragma unroll
      for (int bp = 0; bp < AL_NB / 2; ++bp) {
        const int m = wave + 4 * bp;
        if (m < NGT) *(float2*)(part_o + base * Dv + 32 * m + 2 * fr) = make_float2(o[2 * bp][e], o[2 * bp + 1][e]);
      }
      continue;
    }
    const float l = lfin[hr];
    float f = l > 0.f ? 1.f / l : 0.f;
    if (gate) f *= 1.f / (1.f + __expf(-(float)gate[(long)r * ldg + h]));
#pragma unroll
    for (int bp = 0; bp < AL_NB / 2; ++bp) {
      const int m = wave + 4 * bp;
      if (m < NGT) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const bf16x2 pair = {(bf16)(o[2 * bp][e] * f), (bf16)(o[2 * bp + 1][e] * f)};
        *(bf16x2*)(out + ((long)r * H + h) * Dv + 32 * m + 2 * fr) = pair;
      }
    }
  }
}

// out[row][h][d] = gate * sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the key splits
__global__ __launch_bounds__(128) void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                           int nsplit, int H, int Dv, const bf16* __restrict__ gate, int ldg,
                                                           bf16* __restrict__ out) {
  __shared__ float ws[64];               // weight of every split, e^(m_s - M) / L (times the gate): nsplit <= 64
  __shared__ float red[2];
  const int row = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const long base = ((long)row * H + h) * nsplit;
  float m = -INFINITY, l = 0.f;
  if (tid < nsplit) { m = part_ml[2 * (base + tid)]; l = part_ml[2 * (base + tid) + 1]; }
  // the first wave holds every split (nsplit <= 64): its maximum and weighted sum by wave reductions
  if (tid < 64) {
    const float M = wave_max(m);
    const float w = m == -INFINITY ? 0.f : __expf(m - M);
    const float L = wave_sum(l * w);
    ws[tid] = w;
    if (tid == 0) {
      float f = L > 0.f ? 1.f / L : 0.f;
      if (gate) f *= 1.f / (1.f + __expf(-(float)gate[(long)row * ldg + h]));
      red[0] = f;
    }
  }
  __syncthreads();
  const float f = red[0];
  for (int d = tid; d < Dv; d += 128) {
    float acc = 0.f;
    for (int s = 0; s < nsplit; ++s) acc = fmaf(part_o[(base + s) * Dv + d], ws[s], acc);
    out[((long)row * H + h) * Dv + d] = (bf16)(acc * f);
  }
}

}  // namespace la

// returns 1 when the shape is not this kernel's (the caller runs the row kernel instead)
extern "C" int la_attn_latent(const void* q, const void* kc, const void* row_seq, const void* pos, const void* bt, int maxb,
                              int T, int H, int Dk, int Dv, int BS, float scale, int window, const void* gate, int ldg,
                              void* out, int nsplit, void* part_o, void* part_ml, void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || Dv > Dk || BS <= 0 || !q || !kc || !row_seq || !pos || !bt || !out) return -1;
  if ((Dk & 31) || (Dv & 31) || Dk > 64 * AL_QF || Dv > 64 * AL_NB) return 1;
  if (nsplit < 1 || (nsplit > 1 && (!part_o || !part_ml))) return -2;
  const size_t shm = sizeof(float) * (2 * 16 * AL_SS + 48) + sizeof(bf16) * (16 * AL_PS + (size_t)AL_KT * (Dk + 8));
  if (shm > 64 * 1024) return 1;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(attn_latent_kernel, dim3(T, (H + 15) / 16, nsplit), dim3(256), shm, s, (const bf16*)q, (const bf16*)kc,
                     (const int*)row_seq, (const int*)pos, (const int*)bt, maxb, H, Dk, Dv, BS, scale, window,
                     (const bf16*)gate, ldg, (bf16*)out, nsplit, (float*)part_o, (float*)part_ml);
  int rc = (int)hipGetLastError();
  if (rc || nsplit == 1) return rc ? -10 - rc : 0;
  hipLaunchKernelGGL(latent_merge_kernel, dim3(T, H), dim3(128), 0, s, (const float*)part_o, (const float*)part_ml, nsplit, H,
                     Dv, (const bf16*)gate, ldg, (bf16*)out);
  rc = (int)hipGetLastError();
  return rc ? -10 - rc : 0;
}
