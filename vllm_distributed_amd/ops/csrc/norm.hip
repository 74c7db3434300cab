// RMSNorm family: plain, fused residual-add, and the same two with fp8 output
// (static per-tensor scale, or dynamic per-token scale computed in the same pass).
// One workgroup per token row; the row stays in registers between the two
// passes so HBM is read once.  Reference ops: csrc/layernorm_kernels.cu,
// csrc/layernorm_quant_kernels.cu,
// csrc/quantization/fused_kernels/fused_layernorm_dynamic_per_token_quant.cu.
#include "common.h"

// QUANT: 0 = T out, 1 = fp8 static scale, 2 = fp8 dynamic per-token scale
template <typename T, bool ADD, int QUANT, int MAXV>
__global__ __launch_bounds__(1024) void rms_norm_kernel(
    void* __restrict__ out, const T* __restrict__ in, T* __restrict__ residual, const T* __restrict__ w,
    float eps, int H, long in_stride, long res_stride, long out_stride, float wbias,
    const float* __restrict__ static_scale, float* __restrict__ token_scale, const float* scale_ub) {
  using V8 = typename Vec<T>::v8;
  __shared__ float red[16];
  const long row = blockIdx.x;
  const int nvec = H >> 3;
  const T* ip = in + row * in_stride;
  T* rp = ADD ? residual + row * res_stride : nullptr;
  V8 x[MAXV];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = threadIdx.x + v * blockDim.x;
    if (i < nvec) {
      V8 a = ld16<V8>(ip + 8 * i);
      if (ADD) {
        const V8 b = ld16<V8>(rp + 8 * i);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = (T)((float)a[j] + (float)b[j]);
        st16<V8>(rp + 8 * i, a);
      }
      x[v] = a;
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float f = (float)a[j]; ss += f * f; }
    }
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)H + eps);

  if (QUANT == 0) {
    T* op = (T*)out + row * out_stride;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
      const int i = threadIdx.x + v * blockDim.x;
      if (i < nvec) {
        const V8 ww = ld16<V8>(w + 8 * i);
        V8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          o[j] = (T)((float)(T)((float)x[v][j] * rstd) * ((float)ww[j] + wbias));
        st16<V8>(op + 8 * i, o);
      }
    }
  } else {
    float y[MAXV][8];
    float amax = 0.f;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
      const int i = threadIdx.x + v * blockDim.x;
      if (i < nvec) {
        const V8 ww = ld16<V8>(w + 8 * i);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          y[v][j] = (float)(T)((float)(T)((float)x[v][j] * rstd) * ((float)ww[j] + wbias));
          amax = fmaxf(amax, fabsf(y[v][j]));
        }
      }
    }
    float inv;
    if (QUANT == 2) {
      amax = block_max(amax, red);
      if (scale_ub) amax = fminf(amax, *scale_ub);
      const float sc = fmaxf(amax / 448.f, 1.f / (448.f * 512.f));
      if (threadIdx.x == 0) token_scale[row] = sc;
      inv = 1.f / sc;
    } else {
      inv = 1.f / *static_scale;
    }
    uint8_t* op = (uint8_t*)out + row * out_stride;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
      const int i = threadIdx.x + v * blockDim.x;
      if (i < nvec) {
        u32x2 pk;
        pk[0] = pack_fp8x4(y[v][0] * inv, y[v][1] * inv, y[v][2] * inv, y[v][3] * inv);
        pk[1] = pack_fp8x4(y[v][4] * inv, y[v][5] * inv, y[v][6] * inv, y[v][7] * inv);
        *reinterpret_cast<u32x2*>(op + 8 * i) = pk;
      }
    }
  }
}

template <typename T, bool ADD, int QUANT>
static int launch_norm(void* out, const void* in, void* res, const void* w, float eps, int rows, int H,
                       long in_stride, long res_stride, long out_stride, float wbias, const float* sscale,
                       float* tscale, const float* ub, hipStream_t st) {
  if (H % 8) return -1;
  const int nvec = H / 8;
  int threads = ((nvec + 63) / 64) * 64;
  if (threads > 1024) threads = 1024;
  const int need = (nvec + threads - 1) / threads;
  if (need > 8) return -2;   // H up to 65536
  dim3 grid(rows), block(threads);
#define L(MV) hipLaunchKernelGGL((rms_norm_kernel<T, ADD, QUANT, MV>), grid, block, 0, st, out, (const T*)in, \
                                 (T*)res, (const T*)w, eps, H, in_stride, res_stride, out_stride, wbias, sscale, tscale, ub)
  if (need <= 1) L(1); else if (need <= 2) L(2); else if (need <= 4) L(4); else L(8);
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// quant: 0 none, 1 static fp8, 2 dynamic per-token fp8.  residual may be null.
VDA_EXPORT int vda_rms_norm(void* out, const void* in, void* residual, const void* weight, float eps,
                            int rows, int H, long in_stride, long res_stride, long out_stride,
                            float weight_bias, int quant, const float* static_scale, float* token_scale,
                            const float* scale_ub, int dtype, hipStream_t st) {
#define GO(TT, A, Q) return launch_norm<TT, A, Q>(out, in, residual, weight, eps, rows, H, in_stride, res_stride, \
                                                  out_stride, weight_bias, static_scale, token_scale, scale_ub, st)
#define BYQ(TT, A) do { if (quant == 0) GO(TT, A, 0); else if (quant == 1) GO(TT, A, 1); else GO(TT, A, 2); } while (0)
  if (rows == 0) return 0;
  if (dtype == VDA_BF16) { if (residual) BYQ(bf16_t, true); else BYQ(bf16_t, false); }
  if (dtype == VDA_F16) { if (residual) BYQ(f16_t, true); else BYQ(f16_t, false); }
#undef BYQ
#undef GO
  return -3;
}

// LayerNorm (mean/variance, weight + bias) for OPT / GPT-2 style models.
template <typename T, int MAXV>
__global__ __launch_bounds__(1024) void layer_norm_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                          const T* __restrict__ w, const T* __restrict__ b,
                                                          float eps, int H, long in_stride, long out_stride) {
  using V8 = typename Vec<T>::v8;
  __shared__ float red[16];
  const long row = blockIdx.x;
  const int nvec = H >> 3;
  const T* ip = in + row * in_stride;
  V8 x[MAXV];
  float s = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = threadIdx.x + v * blockDim.x;
    if (i < nvec) {
      x[v] = ld16<V8>(ip + 8 * i);
#pragma unroll
      for (int j = 0; j < 8; ++j) s += (float)x[v][j];
    }
  }
  const float mean = block_sum(s, red) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = threadIdx.x + v * blockDim.x;
    if (i < nvec) {
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float d = (float)x[v][j] - mean; ss += d * d; }
    }
  }
  const float rstd = rsqrtf(block_sum(ss, red) / (float)H + eps);
  T* op = out + row * out_stride;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = threadIdx.x + v * blockDim.x;
    if (i < nvec) {
      const V8 ww = ld16<V8>(w + 8 * i);
      V8 bb = V8{};
      if (b) bb = ld16<V8>(b + 8 * i);
      V8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (T)(((float)x[v][j] - mean) * rstd * (float)ww[j] + (float)bb[j]);
      st16<V8>(op + 8 * i, o);
    }
  }
}

VDA_EXPORT int vda_layer_norm(void* out, const void* in, const void* w, const void* b, float eps, int rows,
                              int H, long in_stride, long out_stride, int dtype, hipStream_t st) {
  if (H % 8) return -1;
  if (rows == 0) return 0;
  const int nvec = H / 8;
  int threads = ((nvec + 63) / 64) * 64;
  if (threads > 1024) threads = 1024;
  const int need = (nvec + threads - 1) / threads;
  if (need > 8) return -2;
  dim3 grid(rows), block(threads);
#define L(TT, MV) hipLaunchKernelGGL((layer_norm_kernel<TT, MV>), grid, block, 0, st, (TT*)out, (const TT*)in, \
                                     (const TT*)w, (const TT*)b, eps, H, in_stride, out_stride)
#define BY(TT) do { if (need <= 1) L(TT, 1); else if (need <= 2) L(TT, 2); else if (need <= 4) L(TT, 4); else L(TT, 8); } while (0)
  if (dtype == VDA_BF16) BY(bf16_t); else if (dtype == VDA_F16) BY(f16_t); else return -3;
#undef BY
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// ---- fp32 residual with a norm after and before every sub-layer ("sandwich" norms) -----------------------------
//   x += y / rms(y) * (off + w_post)      (y given: the output of the sub-layer that just ran)
//   h  = x / rms(x) * (off + w_pre)       (h given: the input of the next sub-layer)
// One pass over the fp32 residual row per token: the write of one sub-layer and the read of the next are one launch,
// the role add + RMSNorm fusion plays for 16-bit residuals.  Gains are fp32; `off` is 1 for gains stored around zero.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void residual_norms_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                             long y_stride, const float* __restrict__ w_post,
                                                             const float* __restrict__ w_pre, T* __restrict__ h,
                                                             long h_stride, float eps, float off, int W) {
  // VEC consecutive values per thread and trip (4: rows whose width and strides are multiples of four)
  extern __shared__ float row[];          // the updated residual row
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  float* xr = x + t * W;
  const T* yr = y ? y + t * y_stride : nullptr;
  float ry = 0.f;
  if (y) {
    float ss = 0.f;
    for (int c = tid * VEC; c < W; c += 256 * VEC) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float v = (float)yr[c + i];
        ss += v * v;
      }
    }
    ss = block_sum(ss, red);
    ry = 1.f / sqrtf(ss / (float)W + eps);
  }
  float sx = 0.f;
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
    float v[VEC];
    if (VEC == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
      v[0] = q[0]; v[1 % VEC] = q[1]; v[2 % VEC] = q[2]; v[3 % VEC] = q[3];
    } else {
      v[0] = xr[c];
    }
    if (y) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] += (float)yr[c + i] * ry * (off + w_post[c + i]);
      if (VEC == 4) *reinterpret_cast<f32x4*>(xr + c) = f32x4{v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]};
      else xr[c] = v[0];
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      row[c + i] = v[i];
      sx += v[i] * v[i];
    }
  }
  if (!h) return;
  sx = block_sum(sx, red);
  const float rx = 1.f / sqrtf(sx / (float)W + eps);
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) h[t * h_stride + c + i] = (T)(row[c + i] * rx * (off + w_pre[c + i]));
  }
}

// y[t, g, :] = x[t, g, :] / rms(x[t, g, :]) * weight[g, :] over `groups` equal parts of a row (fp32 inside)
template <typename T, typename TW>
__global__ __launch_bounds__(256) void group_rms_norm_kernel(T* __restrict__ out, long o_stride,
                                                             const T* __restrict__ x, long x_stride,
                                                             const TW* __restrict__ weight, float eps, int part) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int g = blockIdx.y, tid = threadIdx.x;
  const T* xr = x + t * x_stride + (long)g * part;
  float ss = 0.f;
  for (int c = tid; c < part; c += 256) {
    const float v = (float)xr[c];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)part + eps);
  for (int c = tid; c < part; c += 256)
    out[t * o_stride + (long)g * part + c] = (T)((float)xr[c] * r * (float)weight[(long)g * part + c]);
}

VDA_EXPORT int vda_group_rms_norm(void* out, long o_stride, const void* x, long x_stride, const void* weight,
                                  float eps, int T, int W, int groups, int dtype, int wdtype, hipStream_t st) {
  if (T <= 0) return 0;
  if (groups < 1 || W % groups) return -1;
  dim3 grid(T, groups), block(256);
#define L(TT, TW) hipLaunchKernelGGL((group_rms_norm_kernel<TT, TW>), grid, block, 0, st, (TT*)out, o_stride,       \
                                     (const TT*)x, x_stride, (const TW*)weight, eps, W / groups)
  if (dtype == VDA_BF16 && wdtype == VDA_BF16) L(bf16_t, bf16_t);
  else if (dtype == VDA_BF16 && wdtype == VDA_F32) L(bf16_t, float);
  else if (dtype == VDA_F16 && wdtype == VDA_F16) L(f16_t, f16_t);
  else if (dtype == VDA_F16 && wdtype == VDA_F32) L(f16_t, float);
  else if (dtype == VDA_F32 && wdtype == VDA_F32) L(float, float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// Parallel sub-layers behind per-channel gates over an fp32 residual, and the next norm in groups, in ONE pass:
//   x[t] += sum over the sub-layers of (y + extra_w[t] * extra) * scale * sigmoid(gate)      (in place, fp32)
//   h[t]  = x[t] / rms_g(x[t]) * w_next    with rms_g the root mean square of the value's own part, the row being
//           split into `groups` equal consecutive parts
// Every piece is optional: no sub-layer at all is the stack's first or last norm, no h is the last residual update; up to
// three sub-layer outputs join in one pass (a shared expert beside the routed ones takes the third place).
// One workgroup per token; the updated row waits in LDS for its parts' sums.
struct GatedSub {
  const void* y;        // [T, W] the sub-layer's output
  long y_stride;
  const float* scale;   // [W] or null
  const void* gate;     // [T, W] pre-activations of the sigmoid gate, or null
  long gate_stride;
  const void* extra;    // [T, W] or null: joins y times extra_w[t]
  long extra_stride;
  const float* extra_w; // [T]
};
struct GatedResidualArgs {
  float* x;
  GatedSub sub[3];
  int nsub;
  const float* w_next;
  void* h;
  long h_stride;
  float eps;
  int W, groups;
};

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gated_residual_group_norm_kernel(const GatedResidualArgs a) {
  extern __shared__ float row[];          // the updated residual row, then one factor per part
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = a.W;
  float* xr = a.x + t * W;
  float* rs = row + W;
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
    float v[VEC], add[VEC];
    if (VEC == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
      v[0] = q[0]; v[1 % VEC] = q[1]; v[2 % VEC] = q[2]; v[3 % VEC] = q[3];
    } else {
      v[0] = xr[c];
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) add[i] = 0.f;
    for (int sI = 0; sI < a.nsub; ++sI) {
      const GatedSub& u = a.sub[sI];
      const T* yr = (const T*)u.y + t * u.y_stride + c;
      const T* gr = u.gate ? (const T*)u.gate + t * u.gate_stride + c : nullptr;
      const T* er = u.extra ? (const T*)u.extra + t * u.extra_stride + c : nullptr;
      const float ew = u.extra ? u.extra_w[t] : 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float f = (float)yr[i];
        if (er) f += ew * (float)er[i];
        if (u.scale) f *= u.scale[c + i];
        if (gr) f *= 1.f / (1.f + expf(-(float)gr[i]));
        add[i] += f;
      }
    }
    if (a.nsub > 0) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) v[i] += add[i];
      if (VEC == 4) *reinterpret_cast<f32x4*>(xr + c) = f32x4{v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]};
      else xr[c] = v[0];
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) row[c + i] = v[i];
  }
  if (!a.h) return;
  __syncthreads();
  const int part = W / a.groups;
  for (int g = wave; g < a.groups; g += 4) {
    const float* pr = row + (long)g * part;
    float ss = 0.f;
    for (int c = lane; c < part; c += 64) ss += pr[c] * pr[c];
    ss = wave_sum(ss);
    if (lane == 0) rs[g] = 1.f / sqrtf(ss / (float)part + a.eps);
  }
  __syncthreads();
  T* hr = (T*)a.h + t * a.h_stride;
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) hr[c + i] = (T)(row[c + i] * rs[(c + i) / part] * a.w_next[c + i]);
  }
}

// The same with the row in registers: TRIPS trips of 256 * 4 values cover it.  Either every wave's 256 values of a trip
// lie inside one part (part % 256 == 0): a part's sum of squares is then the sum of whole-wave sums, added up in a
// fixed order by every thread for its own parts (one barrier, no pass through LDS for the row); or a part is 4 * seg
// values for a power of two seg <= 64, i.e. seg neighbouring lanes: its sum comes from shuffles alone.
template <typename T, int TRIPS>
__global__ __launch_bounds__(256) void gated_residual_group_norm_reg_kernel(const GatedResidualArgs a, const int seg) {
  __shared__ float wsum[TRIPS * 4];
  float psum[TRIPS];
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) psum[k] = 0.f;
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int W = a.W;
  float* xr = a.x + t * W;
  float v[TRIPS][4];
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int c = (k * 256 + tid) * 4;
    const bool live = c < W;
    float add[4] = {0.f, 0.f, 0.f, 0.f};
    if (live) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
      v[k][0] = q[0]; v[k][1] = q[1]; v[k][2] = q[2]; v[k][3] = q[3];
      for (int sI = 0; sI < a.nsub; ++sI) {
        const GatedSub& u = a.sub[sI];
        using V4 = typename Vec<T>::v4;
        const V4 y4 = *reinterpret_cast<const V4*>((const T*)u.y + t * u.y_stride + c);
        float f[4] = {(float)y4[0], (float)y4[1], (float)y4[2], (float)y4[3]};
        if (u.extra) {
          const V4 e4 = *reinterpret_cast<const V4*>((const T*)u.extra + t * u.extra_stride + c);
          const float ew = u.extra_w[t];
#pragma unroll
          for (int i = 0; i < 4; ++i) f[i] += ew * (float)e4[i];
        }
        if (u.scale) {
          const f32x4 s4 = *reinterpret_cast<const f32x4*>(u.scale + c);
#pragma unroll
          for (int i = 0; i < 4; ++i) f[i] *= s4[i];
        }
        if (u.gate) {
          const V4 g4 = *reinterpret_cast<const V4*>((const T*)u.gate + t * u.gate_stride + c);
#pragma unroll
          for (int i = 0; i < 4; ++i) f[i] *= 1.f / (1.f + expf(-(float)g4[i]));
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) add[i] += f[i];
      }
      if (a.nsub > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[k][i] += add[i];
        *reinterpret_cast<f32x4*>(xr + c) = f32x4{v[k][0], v[k][1], v[k][2], v[k][3]};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[k][i] = 0.f;
    }
    if (a.h) {
      float ss = v[k][0] * v[k][0] + v[k][1] * v[k][1] + v[k][2] * v[k][2] + v[k][3] * v[k][3];
      if (seg) {                                      // a part is `seg` neighbouring lanes: its sum stays in the wave
        for (int o = seg >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        psum[k] = ss;
      } else {
        ss = wave_sum(ss);
        if (lane == 0) wsum[k * 4 + wave] = ss;
      }
    }
  }
  if (!a.h) return;
  if (!seg) __syncthreads();
  const int part = W / a.groups;
  T* hr = (T*)a.h + t * a.h_stride;
#pragma unroll
  for (int k = 0; k < TRIPS; ++k) {
    const int c = (k * 256 + tid) * 4;
    if (c >= W) continue;
    float ss = psum[k];
    if (!seg) {
      const int g = c / part;
      ss = 0.f;
#pragma unroll
      for (int j = 0; j < TRIPS * 4; ++j)             // chunk j holds the values from j * 256 on
        if ((j * 256) / part == g) ss += wsum[j];
    }
    const float r = 1.f / sqrtf(ss / (float)part + a.eps);
    const f32x4 w4 = *reinterpret_cast<const f32x4*>(a.w_next + c);
    using V4 = typename Vec<T>::v4;
    V4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (T)(v[k][i] * r * w4[i]);
    *reinterpret_cast<V4*>(hr + c) = o;
  }
}

VDA_EXPORT int vda_gated_residual_group_norm(
    float* x, int nsub, const void* y0, long y0_stride, const float* s0, const void* g0, long g0_stride,
    const void* e0, long e0_stride, const float* ew0, const void* y1, long y1_stride, const float* s1, const void* g1,
    long g1_stride, const void* e1, long e1_stride, const float* ew1, const void* y2, long y2_stride, const float* s2,
    const void* g2, long g2_stride, const void* e2, long e2_stride, const float* ew2, const float* w_next, void* h,
    long h_stride, float eps, int groups, int T, int W, int dtype, hipStream_t st) {
  if (T <= 0 || (nsub == 0 && !h)) return 0;
  if (nsub < 0 || nsub > 3 || (nsub > 0 && !y0) || (nsub > 1 && !y1) || (nsub > 2 && !y2) || (h && !w_next) ||
      groups < 1 || W % groups || (e0 && !ew0) || (e1 && !ew1) || (e2 && !ew2))
    return -1;
  const size_t lds = ((size_t)W + groups) * 4;
  if (lds > 60 * 1024) return -2;
  GatedResidualArgs a;
  a.x = x; a.nsub = nsub; a.w_next = w_next; a.h = h; a.h_stride = h_stride; a.eps = eps; a.W = W; a.groups = groups;
  a.sub[0] = GatedSub{y0, y0_stride, s0, g0, g0_stride, e0, e0_stride, ew0};
  a.sub[1] = GatedSub{y1, y1_stride, s1, g1, g1_stride, e1, e1_stride, ew1};
  a.sub[2] = GatedSub{y2, y2_stride, s2, g2, g2_stride, e2, e2_stride, ew2};
  bool vec = W % 4 == 0 && h_stride % 4 == 0;
  for (int i = 0; i < nsub; ++i)
    vec = vec && a.sub[i].y_stride % 4 == 0 && a.sub[i].gate_stride % 4 == 0 && a.sub[i].extra_stride % 4 == 0;
  // rows of up to 4096 values whose parts are whole numbers of 256-value wave chunks stay in registers
  const int trips = (W + 1023) / 1024;
  const uintptr_t al = dtype == VDA_F32 ? 16 : 8;          // four values of the activation type
  const int part = W / groups;
  int seg = 0;                                             // lanes per part when a part is a power of two <= 256
  if (part % 256 != 0 && part >= 4 && part <= 256 && (part & (part - 1)) == 0) seg = part / 4;
  const bool reg = vec && trips <= 4 && (part % 256 == 0 || seg) && ((uintptr_t)x % 16 == 0) &&
                   (!w_next || (uintptr_t)w_next % 16 == 0) && (!h || (uintptr_t)h % al == 0) && [&] {
                     for (int i = 0; i < nsub; ++i) {
                       const GatedSub& u = a.sub[i];
                       if ((uintptr_t)u.y % al || (uintptr_t)u.gate % al || (uintptr_t)u.extra % al ||
                           (uintptr_t)u.scale % 16)
                         return false;
                     }
                     return true;
                   }();
#define LR(TT, KK) hipLaunchKernelGGL((gated_residual_group_norm_reg_kernel<TT, KK>), dim3(T), dim3(256), 0, st, a, seg)
#define L2(TT, VV) hipLaunchKernelGGL((gated_residual_group_norm_kernel<TT, VV>), dim3(T), dim3(256), lds, st, a)
#define L(TT)                                                                                                       \
  do {                                                                                                              \
    if (reg && trips == 1) LR(TT, 1); else if (reg && trips == 2) LR(TT, 2); else if (reg && trips == 3) LR(TT, 3); \
    else if (reg) LR(TT, 4); else if (vec) L2(TT, 4); else L2(TT, 1);                                               \
  } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
#undef LR
  VDA_CHECK_LAUNCH();
  return 0;
}

VDA_EXPORT int vda_residual_norms(float* x, const void* y, long y_stride, const float* w_post, const float* w_pre,
                                  void* h, long h_stride, float eps, float off, int T, int W, int dtype,
                                  hipStream_t st) {
  if (T <= 0 || (!y && !h)) return 0;
  if ((y && !w_post) || (h && !w_pre)) return -1;
  const size_t lds = (size_t)W * 4;
  if (lds > 60 * 1024) return -2;
  const bool vec = W % 4 == 0 && y_stride % 4 == 0 && h_stride % 4 == 0;
#define L2(TT, VV) hipLaunchKernelGGL((residual_norms_kernel<TT, VV>), dim3(T), dim3(256), lds, st, x, (const TT*)y, \
                                      y_stride, w_post, w_pre, (TT*)h, h_stride, eps, off, W)
#define L(TT) do { if (vec) L2(TT, 4); else L2(TT, 1); } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
#undef L3
  VDA_CHECK_LAUNCH();
  return 0;
}

// fp32 residual whose sub-layers are normed on their OUTPUT: x += (y - mean(y)) / sqrt(var(y) + eps) * w + b, in place,
// and the updated row goes out once more in the activation type, as the next sub-layer's input (one launch for the
// norm, the residual sum and the cast).  Without y: h = layer norm of x itself (the model's last norm), x stays.
// With y2 and gate the sub-layer's output is y + y2 * sigmoid(gate[t]) (a shared expert behind its gate), formed here.
// The source row sits in LDS between the passes (mean, squared deviations, output).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void residual_layer_norm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                  long y_stride, const float* __restrict__ w,
                                                                  const float* __restrict__ b, T* __restrict__ h,
                                                                  long h_stride, float eps, int W,
                                                                  const T* __restrict__ y2, long y2_stride,
                                                                  const float* __restrict__ gate, long gate_stride) {
  // VEC consecutive values per thread and trip (4: rows whose width and strides are multiples of four, moved as
  // 16-byte fp32 / 8- or 16-byte activation vectors)
  using V4 = typename Vec<T>::v4;
  extern __shared__ float row[];
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int tid = threadIdx.x;
  float* xr = x + t * W;
  const T* yr = y ? y + t * y_stride : nullptr;
  // a second part of the sub-layer's output behind a sigmoid gate of one number per row: y + y2 * sigmoid(gate[t])
  const T* y2r = (y && y2) ? y2 + t * y2_stride : nullptr;
  const float g2 = y2r ? 1.f / (1.f + expf(-gate[t * gate_stride])) : 0.f;
  float s = 0.f;
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
    float v[VEC];
    if (VEC == 4) {
      if (yr) {
        const V4 q = *reinterpret_cast<const V4*>(yr + c);
        v[0] = (float)q[0]; v[1 % VEC] = (float)q[1]; v[2 % VEC] = (float)q[2]; v[3 % VEC] = (float)q[3];
        if (y2r) {
          const V4 q2 = *reinterpret_cast<const V4*>(y2r + c);
          v[0] += g2 * (float)q2[0]; v[1 % VEC] += g2 * (float)q2[1]; v[2 % VEC] += g2 * (float)q2[2];
          v[3 % VEC] += g2 * (float)q2[3];
        }
      } else {
        const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
        v[0] = q[0]; v[1 % VEC] = q[1]; v[2 % VEC] = q[2]; v[3 % VEC] = q[3];
      }
      *reinterpret_cast<f32x4*>(row + c) = f32x4{v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]};
    } else {
      v[0] = yr ? (float)yr[c] + (y2r ? g2 * (float)y2r[c] : 0.f) : xr[c];
      row[c] = v[0];
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) s += v[i];
  }
  const float mean = block_sum(s, red) / (float)W;
  float ss = 0.f;
  for (int c = tid * VEC; c < W; c += 256 * VEC) {       // a thread re-reads what it wrote itself
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float d = row[c + i] - mean;
      ss += d * d;
    }
  }
  const float r = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
  for (int c = tid * VEC; c < W; c += 256 * VEC) {
    float v[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = (row[c + i] - mean) * r * w[c + i] + (b ? b[c + i] : 0.f);
    if (VEC == 4) {
      if (yr) {
        const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
        v[0] += q[0]; v[1 % VEC] += q[1]; v[2 % VEC] += q[2]; v[3 % VEC] += q[3];
        *reinterpret_cast<f32x4*>(xr + c) = f32x4{v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]};
      }
      if (h) {
        V4 o;
        o[0] = (T)v[0]; o[1] = (T)v[1 % VEC]; o[2] = (T)v[2 % VEC]; o[3] = (T)v[3 % VEC];
        *reinterpret_cast<V4*>(h + t * h_stride + c) = o;
      }
    } else {
      if (yr) {
        v[0] += xr[c];
        xr[c] = v[0];
      }
      if (h) h[t * h_stride + c] = (T)v[0];
    }
  }
}

VDA_EXPORT int vda_residual_layer_norm(float* x, const void* y, long y_stride, const float* w, const float* b,
                                       void* h, long h_stride, float eps, int T, int W, int dtype, const void* y2,
                                       long y2_stride, const float* gate, long gate_stride, hipStream_t st) {
  if (T <= 0) return 0;
  if (!w || (!y && !h) || (y2 && (!y || !gate))) return -1;
  const size_t lds = (size_t)W * 4;
  if (lds > 60 * 1024) return -2;
  const bool vec = W % 4 == 0 && y_stride % 4 == 0 && h_stride % 4 == 0 && y2_stride % 4 == 0;
#define L2(TT, VV) hipLaunchKernelGGL((residual_layer_norm_kernel<TT, VV>), dim3(T), dim3(256), lds, st, x,          \
                                      (const TT*)y, y_stride, w, b, (TT*)h, h_stride, eps, W, (const TT*)y2,          \
                                      y2_stride, gate, gate_stride)
#define L(TT) do { if (vec) L2(TT, 4); else L2(TT, 1); } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
#undef L3
  VDA_CHECK_LAUNCH();
  return 0;
}

// Dot products that a design wants in fp32 although the activations are 16-bit: out[t, r] = bias[r] + x[t, :] . w[r, :]
// with fp32 weights (router logits, one-number gates).  A wave takes 8 tokens: per 512-column step it holds 8 weight
// rows x 8 columns per lane in registers and streams the 8 tokens' values past them (16-byte loads), so weights come
// from cache once per 8 tokens and every activation row is read once per group of 8 output rows; the 64 partial sums
// are reduced over the lanes at the end.  Widths that are not a multiple of 8 take one value per lane and step.
template <typename T, bool VEC, int TT>
__global__ __launch_bounds__(256) void fp32_rows_dot_kernel(float* __restrict__ out, const T* __restrict__ x,
                                                            long x_stride, const float* __restrict__ w,
                                                            const float* __restrict__ bias, int T_, int R, int W) {
  using V8 = typename Vec<T>::v8;
  constexpr int RR = 8, CL = VEC ? 8 : 1;       // rows per pass, columns per lane and step (TT: tokens per wave)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long t0 = ((long)blockIdx.x * 4 + wave) * TT;
  if (t0 >= T_) return;
  for (int r0 = 0; r0 < R; r0 += RR) {
    float acc[TT][RR];
#pragma unroll
    for (int a = 0; a < TT; ++a)
#pragma unroll
      for (int b = 0; b < RR; ++b) acc[a][b] = 0.f;
    for (int c0 = lane * CL; c0 < W; c0 += 64 * CL) {
      float wr[RR][CL];
#pragma unroll
      for (int b = 0; b < RR; ++b) {
        const float* wp = w + (long)min(r0 + b, R - 1) * W + c0;
#pragma unroll
        for (int i = 0; i < CL; ++i) wr[b][i] = wp[i];
      }
#pragma unroll
      for (int a = 0; a < TT; ++a) {
        const T* xp = x + min(t0 + a, (long)T_ - 1) * x_stride + c0;
        float xv[CL];
        if (VEC) {
          const V8 v = ld16<V8>(xp);
#pragma unroll
          for (int i = 0; i < CL; ++i) xv[i] = (float)v[i];
        } else {
          xv[0] = (float)xp[0];
        }
#pragma unroll
        for (int b = 0; b < RR; ++b)
#pragma unroll
          for (int i = 0; i < CL; ++i) acc[a][b] += xv[i] * wr[b][i];
      }
    }
    if (TT * RR == 64) {
      // 64 sums over 64 lanes in 63 exchanges instead of 64 x 6: at every step a lane keeps one half of its values and
      // hands the other half to its partner; in the end lane L holds the total of value L = (token L / 8, row L % 8)
      float* f = &acc[0][0];
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) {
        const bool up = lane & o;
#pragma unroll
        for (int i = 0; i < o; ++i) {
          const float keep = up ? f[i + o] : f[i], give = up ? f[i] : f[i + o];
          f[i] = keep + __shfl_xor(give, o, 64);
        }
      }
      const int a = lane / RR, b = lane % RR;
      if (t0 + a < T_ && r0 + b < R) out[(t0 + a) * R + r0 + b] = f[0] + (bias ? bias[r0 + b] : 0.f);
    } else {
#pragma unroll
      for (int a = 0; a < TT; ++a)
#pragma unroll
        for (int b = 0; b < RR; ++b) {
          const float v = wave_sum(acc[a][b]);
          if (lane == 0 && t0 + a < T_ && r0 + b < R) out[(t0 + a) * R + r0 + b] = v + (bias ? bias[r0 + b] : 0.f);
        }
    }
  }
}

VDA_EXPORT int vda_fp32_rows_dot(float* out, const void* x, long x_stride, const float* w, const float* bias, int T,
                                 int R, int W, int dtype, hipStream_t st) {
  if (T <= 0 || R <= 0) return 0;
  const bool vec = W % 8 == 0 && x_stride % 8 == 0 && (uintptr_t)x % 32 == 0;
  const bool many = T >= 4096;          // few tokens (decoding): one per wave, for the launch to spread over the chip
  const dim3 grid((unsigned)(many ? (T + 31) / 32 : (T + 3) / 4)), block(256);
#define L3(TT, VV, NT) hipLaunchKernelGGL((fp32_rows_dot_kernel<TT, VV, NT>), grid, block, 0, st, out, (const TT*)x,   \
                                          x_stride, w, bias, T, R, W)
#define L2(TT, VV) do { if (many) L3(TT, VV, 8); else L3(TT, VV, 1); } while (0)
#define L(TT) do { if (vec) L2(TT, true); else L2(TT, false); } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
#undef L3
  VDA_CHECK_LAUNCH();
  return 0;
}
