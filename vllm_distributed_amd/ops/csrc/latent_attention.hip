// Latent attention over a sliding window, on a paged cache of latent rows, for any sizes.
//
// The cache keeps ONE row per token, kc [blocks, bs, DK] with DK = R + P: the normalised latent c (R values) followed
// by a rotated key part shared by all heads (P values).  Queries arrive with the key up-projection folded in
// (qf[t, h] = [W_uk_h^T q_nope | rotated q_rot]), so every head dots against the same rows, and the output stays in
// latent space (sum of weights * c) for the caller's value up-projection.
//
//   vda_latent_norm_rope_cache   per token: c = down[:R] / rms * weight, rotate down[R:] and every query head's last
//                                P values (interleaved pairs, angles from an fp32 cos | sin table), write the cache
//                                row (and, for the MFMA kernel of mla.hip, the transposed copy of c) and
//                                qf[:, :, R:] in one launch
//   vda_latent_window_attention  softmax(scale * qf . row) over the keys j <= i, i - j < window (with `sink`, exp(sink[h])
//                                joins head h's denominator without key or value); scores, softmax and
//                                the weighted sum in fp32.  One workgroup per (sequence, tile of query tokens) walks
//                                the visible keys in tiles through LDS with a running maximum and sum per row; keys
//                                outside the window are never loaded.  Prompts, portions and single decoded tokens
//                                are one code path; keys are added in a fixed order per (token, head).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void latent_norm_rope_cache_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ down, long down_stride,
    const float* __restrict__ c_weight, const float* __restrict__ cos_sin, const long* __restrict__ positions,
    T* __restrict__ qf, T* __restrict__ kc, T* __restrict__ vt, const long* __restrict__ slot_mapping, int H, int D,
    int P, int R, int rot, int bs, float eps) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  const int DK = R + P, half = rot / 2;
  const T* dr = down + t * down_stride;
  const float* cs = cos_sin + positions[t] * (long)rot;
  float ss = 0.f;
  for (int c = tid; c < R; c += 256) {
    const float v = (float)dr[c];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)R + eps);
  const long slot = slot_mapping[t];
  T* row = slot >= 0 ? kc + slot * (long)DK : nullptr;      // slot = block * bs + offset, rows are contiguous
  if (row) {
    T* col = vt ? vt + ((slot / bs) * R) * (long)bs + slot % bs : nullptr;     // vt [blocks, R, bs]
    for (int c = tid; c < R; c += 256) {
      const T v = (T)((float)dr[c] * rs * c_weight[c]);
      row[c] = v;
      if (col) col[(long)c * bs] = v;
    }
    for (int i = tid; i < P; i += 256) {
      float v;
      if (i < rot) {
        const int pr = i >> 1;
        const float co = cs[pr], si = cs[half + pr];
        const float u = (float)dr[R + (i & ~1)], w = (float)dr[R + (i | 1)];
        v = (i & 1) ? w * co + u * si : u * co - w * si;
      } else {
        v = (float)dr[R + i];
      }
      row[R + i] = (T)v;
    }
  }
  // the query heads' rotated parts
  for (int e = tid; e < H * P; e += 256) {
    const int h = e / P, i = e % P;
    const T* qp = q + t * q_stride + (long)h * (D + P) + D;
    float v;
    if (i < rot) {
      const int pr = i >> 1;
      const float co = cs[pr], si = cs[half + pr];
      const float u = (float)qp[i & ~1], w = (float)qp[i | 1];
      v = (i & 1) ? w * co + u * si : u * co - w * si;
    } else {
      v = (float)qp[i];
    }
    qf[(t * H + h) * DK + R + i] = (T)v;
  }
}

VDA_EXPORT int vda_latent_norm_rope_cache(const void* q, long q_stride, const void* down, long down_stride,
                                          const float* c_weight, const float* cos_sin, const long* positions,
                                          void* qf, void* kc, void* vt, const long* slot_mapping, int T, int H, int D,
                                          int P, int R, int rot, int bs, float eps, int dtype, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > P || (rot & 1)) return -1;
#define L(TT) hipLaunchKernelGGL((latent_norm_rope_cache_kernel<TT>), dim3(T), dim3(256), 0, st, (const TT*)q,      \
                                 q_stride, (const TT*)down, down_stride, c_weight, cos_sin, positions, (TT*)qf,      \
                                 (TT*)kc, (TT*)vt, slot_mapping, H, D, P, R, rot, bs, eps)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// NACC: output values per thread (BQ * H * R <= 256 * NACC); M = BQ * H query rows per workgroup (at most 256)
template <typename T, int NACC>
__global__ __launch_bounds__(256) void latent_window_attention_kernel(
    T* __restrict__ out, const T* __restrict__ qf, const T* __restrict__ kc, const int* __restrict__ block_table,
    long bt_stride, const int* __restrict__ seq_lens, const int* __restrict__ qsl, float scale, int window, int HT,
    int HG, int DK, int R, int bs, int BQ, int BK, const float* __restrict__ sink) {
  // HT heads in all; this workgroup takes the H heads from h0 on (grid.z deals groups of HG heads)
  const int h0 = blockIdx.z * HG;
  const int H = min(HG, HT - h0);
  extern __shared__ float lds[];
  const int Dq = (DK + 3) / 4 * 4 + 1;          // padded row of q and the latent rows (odd: no bank conflicts
  const int RS = BK + 1;                        //  when lanes walk rows)
  const int M = BQ * H;
  float* qs = lds;                              // [M][Dq]
  float* ks = qs + M * Dq;                      // [BK][Dq]
  float* sc = ks + BK * Dq;                     // [M][RS] scores, then weights
  float* rm = sc + M * RS;                      // [M] running maximum
  float* rl = rm + M;                           // [M] running sum
  float* ra = rl + M;                           // [M] rescale of this tile

  const int s = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  const int i0 = blockIdx.x * BQ;
  if (i0 >= L) return;
  const int nq = min(BQ, L - i0);
  const int p0 = sl - L + i0, p1 = p0 + nq;      // positions of the tile's queries: [p0, p1)
  const int* bt = block_table + (long)s * bt_stride;

  for (int e = tid; e < M * DK; e += 256) {
    const int d = e % DK, m = e / DK;             // m = i * H + h
    qs[m * Dq + d] = (m / H) < nq ? (float)qf[((long)(t0 + i0 + m / H) * HT + h0 + m % H) * DK + d] * scale : 0.f;
  }
  for (int m = tid; m < M; m += 256) {
    if (sink) { rm[m] = sink[h0 + m % H]; rl[m] = 1.f; }        // exp(sink - sink): the sink's share of the sum
    else { rm[m] = -INFINITY; rl[m] = 0.f; }
  }
  float acc[NACC];
#pragma unroll
  for (int n = 0; n < NACC; ++n) acc[n] = 0.f;

  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int ntiles = (p1 - lo + BK - 1) / BK;
  for (int tile = 0; tile < ntiles; ++tile) {
    const int j0 = lo + tile * BK;
    const int nk = min(BK, p1 - j0);
    __syncthreads();
    for (int e = tid; e < BK * DK; e += 256) {
      const int d = e % DK, jj = e / DK;
      float v = 0.f;
      if (jj < nk) {
        const int j = j0 + jj;
        v = (float)kc[((long)bt[j / bs] * bs + j % bs) * DK + d];
      }
      ks[jj * Dq + d] = v;
    }
    __syncthreads();
    for (int e = tid; e < M * BK; e += 256) {
      const int jj = e % BK, m = e / BK;
      const int pi = p0 + m / H, j = j0 + jj;
      float a = -INFINITY;
      if (m / H < nq && jj < nk && j <= pi && (window <= 0 || pi - j < window)) {
        const float* qp = qs + m * Dq;
        const float* kp = ks + jj * Dq;
        a = 0.f;
        for (int d = 0; d < DK; ++d) a += qp[d] * kp[d];
      }
      sc[m * RS + jj] = a;
    }
    __syncthreads();
    // running maximum and sum per row; scores become weights relative to the new maximum
    for (int m = tid; m < M; m += 256) {
      float* sp = sc + m * RS;
      float mx = rm[m];
      for (int jj = 0; jj < nk; ++jj) mx = fmaxf(mx, sp[jj]);
      const float mu = mx == -INFINITY ? 0.f : mx;
      const float al = expf(rm[m] - mu);        // rm = -inf: 0
      float sum = 0.f;
      for (int jj = 0; jj < nk; ++jj) {
        const float w = expf(sp[jj] - mu);
        sp[jj] = w;
        sum += w;
      }
      rm[m] = mx;
      rl[m] = rl[m] * al + sum;
      ra[m] = al;
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NACC; ++n) {
      const int e = tid + n * 256;
      if (e < M * R) {
        const int d = e % R, m = e / R;
        const float* wp = sc + m * RS;
        const float* vp = ks + d;
        float a = acc[n] * ra[m];
        for (int jj = 0; jj < nk; ++jj) a += wp[jj] * vp[jj * Dq];
        acc[n] = a;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = tid + n * 256;
    if (e < M * R) {
      const int d = e % R, m = e / R;
      if (m / H < nq) {
        const float l = rl[m];
        out[((long)(t0 + i0 + m / H) * HT + h0 + m % H) * R + d] = (T)(l > 0.f ? acc[n] / l : 0.f);
      }
    }
  }
}

VDA_EXPORT int vda_latent_window_attention(void* out, const void* qf, const void* kc, const int* block_table,
                                           long bt_stride, const int* seq_lens, const int* qsl, float scale,
                                           int window, int S, int H, int DK, int R, int bs, int max_q,
                                           const float* sink, int dtype, hipStream_t st) {
  if (S <= 0 || max_q <= 0) return 0;
  if (H <= 0 || R <= 0 || R > DK) return -1;
  // tile sizes: the largest query tile (then key tile) whose accumulators fit 64 registers per thread, whose rows
  // fit one workgroup and whose tiles fit 96 KiB of LDS; single decoded tokens take a one-token tile; heads are
  // dealt to several workgroups when one token's heads alone are too many for that
  const int Dq = (DK + 3) / 4 * 4 + 1;
  auto lds_of = [&](int bq, int bk, int hg) {
    return ((size_t)bq * hg * Dq + (size_t)bk * Dq + (size_t)bq * hg * (bk + 1) + 3 * (size_t)bq * hg) * 4;
  };
  int BQ = 0, BK = 0, HG = H;
  for (; HG >= 1 && !BQ; HG = HG > 1 ? (HG + 1) / 2 : 0) {
    for (int bq = 16; bq >= 1 && !BQ; bq >>= 1) {
      if (bq > 1 && bq / 2 >= max_q) continue;
      if ((size_t)bq * HG * R > 256 * 64 || bq * HG > 256) continue;
      for (int bk = 64; bk >= 8; bk >>= 1)
        if (lds_of(bq, bk, HG) <= 96 * 1024) { BQ = bq; BK = bk; break; }
    }
    if (BQ) break;
  }
  if (!BQ) return -2;
  const size_t lds = lds_of(BQ, BK, HG);
  const int per = (BQ * HG * R + 255) / 256;
  const int NACC = per <= 8 ? 8 : per <= 16 ? 16 : per <= 32 ? 32 : 64;
  dim3 grid((max_q + BQ - 1) / BQ, S, (H + HG - 1) / HG), block(256);
#define L2(TT, NA)                                                                                                  \
  do {                                                                                                              \
    if (lds > 48 * 1024) {                                                                                          \
      hipError_t e = hipFuncSetAttribute((const void*)latent_window_attention_kernel<TT, NA>,                       \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
      if (e != hipSuccess) return (int)e;                                                                           \
    }                                                                                                               \
    hipLaunchKernelGGL((latent_window_attention_kernel<TT, NA>), grid, block, lds, st, (TT*)out, (const TT*)qf,     \
                       (const TT*)kc, block_table, bt_stride, seq_lens, qsl, scale, window, H, HG, DK, R, bs, BQ,   \
                       BK, sink);                                                                                   \
  } while (0)
#define L(TT)                                                                                                       \
  do {                                                                                                              \
    if (NACC == 8) L2(TT, 8); else if (NACC == 16) L2(TT, 16); else if (NACC == 32) L2(TT, 32); else L2(TT, 64);    \
  } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
  VDA_CHECK_LAUNCH();
  return 0;
}
