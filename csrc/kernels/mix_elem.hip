// Row kernels of the layer-list models: scaled embedding + sinusoid, sandwich norm
// (residual update with the sublayer's output norm and layer scale, fused with the next
// sublayer's input norm), short causal input convolution with per-sequence state,
// per-head q / k / v norms with paged-cache append and query mixing, clamped GLU.
//
// All of them are memory bound: one workgroup per token row, every row read once.
// Norms and the residual stream are fp32 whatever the activation type T is.
#include "mix_common.h"

namespace rfqmix {

// out[t] = table[ids[t]] * scale + pe(pos[t]);  pe[2i] = sin(pos * inv_freq[i]),
// pe[2i+1] = cos(pos * inv_freq[i]).  out is the fp32 residual stream.
template <typename T>
__global__ __launch_bounds__(256) void embed_sinusoid_kernel(
    const int32_t* __restrict__ ids, const int32_t* __restrict__ pos, const T* __restrict__ table,
    const float* __restrict__ inv_freq, float scale, float* __restrict__ out, int d, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (int64_t)id * d;
  const float p = (float)pos[t];
  float* o = out + (int64_t)t * d;
  for (int i = threadIdx.x; 2 * i < d; i += blockDim.x) {
    float sn, cs;
    sincosf(p * inv_freq[i], &sn, &cs);
    o[2 * i] = ldf(row + 2 * i) * scale + sn;
    if (2 * i + 1 < d) o[2 * i + 1] = ldf(row + 2 * i + 1) * scale + cs;
  }
}

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                     __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
  bf16_t t[4];
  stf(t, v.x); stf(t + 1, v.y); stf(t + 2, v.z); stf(t + 3, v.w);
  *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(t);
}

__device__ __forceinline__ void ld8(const float* p, float* f) {
  const float4 a = ld4(p), b = ld4(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void ld8(const bf16_t* p, float* f) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    f[2 * k] = __uint_as_float(w[k] << 16);
    f[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
  }
}
__device__ __forceinline__ void st8(float* p, const float* f) {
  st4(p, make_float4(f[0], f[1], f[2], f[3]));
  st4(p + 4, make_float4(f[4], f[5], f[6], f[7]));
}
__device__ __forceinline__ void st8(bf16_t* p, const float* f) {
  bf16_t t[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) stf(t + k, f[k]);
  *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(t);
}

// The same with the row held in registers: d a multiple of 4, at most NCH * 1024.  Every
// operand is read once, in 16-byte pieces, before the first reduction.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void sandwich_norm_vec_kernel(
    const T* __restrict__ y, int64_t y_stride, float* __restrict__ residual,
    const float* __restrict__ w_post, const float* __restrict__ gain,
    const float* __restrict__ w_pre, float* __restrict__ out, int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* x = residual + (int64_t)t * d;
  float4 xv[NCH], yv[NCH], wn[NCH];
  float sy = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < d) {
      xv[k] = ld4(x + c);
      wn[k] = ld4(w_pre + c);
      if (y != nullptr) {
        const float4 a = ld4(y + (int64_t)t * y_stride + c), p = ld4(w_post + c), g = ld4(gain + c);
        sy += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
        yv[k] = make_float4(a.x * p.x * g.x, a.y * p.y * g.y, a.z * p.z * g.z, a.w * p.w * g.w);
      }
    }
  }
  float ss = 0.f;
  if (y != nullptr) {
    sy = block_sum(sy, scratch);
    const float ry = 1.0f / sqrtf(sy / (float)d + eps);
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int c = (threadIdx.x + k * 256) * 4;
      if (c < d) {
        xv[k].x += yv[k].x * ry; xv[k].y += yv[k].y * ry;
        xv[k].z += yv[k].z * ry; xv[k].w += yv[k].w * ry;
        st4(x + c, xv[k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < NCH; ++k)
    if ((threadIdx.x + k * 256) * 4 < d)
      ss += xv[k].x * xv[k].x + xv[k].y * xv[k].y + xv[k].z * xv[k].z + xv[k].w * xv[k].w;
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)d + eps);
  float* o = out + (int64_t)t * d;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < d)
      st4(o + c, make_float4(xv[k].x * r * wn[k].x, xv[k].y * r * wn[k].y, xv[k].z * r * wn[k].z,
                             xv[k].w * r * wn[k].w));
  }
}

// residual += rms(y) * w_post * gain (when y != nullptr); out = rms(residual) * w_pre.
template <typename T>
__global__ __launch_bounds__(256) void sandwich_norm_kernel(
    const T* __restrict__ y, int64_t y_stride, float* __restrict__ residual,
    const float* __restrict__ w_post, const float* __restrict__ gain,
    const float* __restrict__ w_pre, float* __restrict__ out, int d, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* x = residual + (int64_t)t * d;
  float ss = 0.f;
  if (y != nullptr) {
    const T* yr = y + (int64_t)t * y_stride;
    float sy = 0.f;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
      const float v = ldf(yr + c);
      sy += v * v;
    }
    sy = block_sum(sy, scratch);
    const float ry = 1.0f / sqrtf(sy / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
      const float v = x[c] + ldf(yr + c) * ry * w_post[c] * gain[c];
      x[c] = v;
      ss += v * v;
    }
  } else {
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
      const float v = x[c];
      ss += v * v;
    }
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)d + eps);
  float* o = out + (int64_t)t * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = x[c] * r * w_pre[c];   // own writes
}

// out[t] = h[t] + sum_dl w[:, taps-1-dl] * h(position of t - dl).  Rows of one sequence are
// contiguous; row_back = index inside the scheduled run, row_fwd = rows of the run after it,
// row_state = slot * 2 + half to read (-1: no state).  Inputs before the run come from the
// read half (entry e holds the input at run start - (taps-1) + e), inputs before position 0
// are zero; the run's last taps-1 inputs go to the other half.
template <typename T>
__global__ __launch_bounds__(256) void canon_conv_kernel(
    const float* __restrict__ h, const float* __restrict__ w, float* __restrict__ state,
    const int32_t* __restrict__ row_state, const int32_t* __restrict__ row_back,
    const int32_t* __restrict__ row_fwd, const int32_t* __restrict__ pos, T* __restrict__ out,
    int d, int taps, int slots) {
  const int t = blockIdx.x;
  const int code = row_state[t], i = row_back[t], f = row_fwd[t], p = pos[t];
  const int K = taps - 1;
  const float* rd = code >= 0 ? state + ((int64_t)((code & 1) * slots + (code >> 1)) * K) * d : nullptr;
  float* wr = code >= 0 ? state + ((int64_t)((1 - (code & 1)) * slots + (code >> 1)) * K) * d : nullptr;
  const float* hr = h + (int64_t)t * d;
  const int q = i + f + 1;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float h0 = hr[c];
    const float* wc = w + (int64_t)c * taps;
    float acc = h0 + wc[taps - 1] * h0;
    for (int dl = 1; dl < taps; ++dl) {
      float src;
      if (dl <= i) src = hr[c - (int64_t)dl * d];
      else if (p - dl >= 0 && rd != nullptr) src = rd[(int64_t)(K + i - dl) * d + c];
      else continue;
      acc += wc[taps - 1 - dl] * src;
    }
    stf(out + (int64_t)t * d + c, acc);
    if (wr != nullptr) {
      if (f < K) wr[(int64_t)(K - 1 - f) * d + c] = h0;
      if (i == 0)
        for (int e = 0; e < K - q; ++e) wr[(int64_t)e * d + c] = rd[(int64_t)(e + q) * d + c];
    }
  }
}

constexpr int kVecTaps = 4;      // most taps of the vector form (compiled per tap count)

// Four channels per thread (d a multiple of 4, at most kVecTaps taps): 16-byte loads of h,
// of the state and of the taps.
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void canon_conv_vec_kernel(
    const float* __restrict__ h, const float* __restrict__ w, float* __restrict__ state,
    const int32_t* __restrict__ row_state, const int32_t* __restrict__ row_back,
    const int32_t* __restrict__ row_fwd, const int32_t* __restrict__ pos, T* __restrict__ out,
    int d, int slots) {
  constexpr int taps = TAPS;
  const int t = blockIdx.x;
  const int code = row_state[t], i = row_back[t], f = row_fwd[t], p = pos[t];
  const int K = taps - 1;
  const float* rd = code >= 0 ? state + ((int64_t)((code & 1) * slots + (code >> 1)) * K) * d : nullptr;
  float* wr = code >= 0 ? state + ((int64_t)((1 - (code & 1)) * slots + (code >> 1)) * K) * d : nullptr;
  const float* hr = h + (int64_t)t * d;
  const int q = i + f + 1;
  for (int c = threadIdx.x * 4; c < d; c += blockDim.x * 4) {
    const float4 h0 = ld4(hr + c);
    // the four channels' taps are 4 * taps contiguous floats: read them in 16-byte pieces
    float wv[4 * TAPS];
#pragma unroll
    for (int k = 0; k < TAPS; ++k)
      *reinterpret_cast<float4*>(wv + 4 * k) = ld4(w + (int64_t)c * taps + 4 * k);
    const float* wc = wv;                                // [4][taps]
    float4 acc = make_float4(h0.x + wc[taps - 1] * h0.x, h0.y + wc[2 * taps - 1] * h0.y,
                             h0.z + wc[3 * taps - 1] * h0.z, h0.w + wc[4 * taps - 1] * h0.w);
#pragma unroll
    for (int dl = 1; dl < taps; ++dl) {
      float4 src;
      if (dl <= i) src = ld4(hr + c - (int64_t)dl * d);
      else if (p - dl >= 0 && rd != nullptr) src = ld4(rd + (int64_t)(K + i - dl) * d + c);
      else continue;
      const int j = taps - 1 - dl;
      acc.x += wc[j] * src.x; acc.y += wc[taps + j] * src.y;
      acc.z += wc[2 * taps + j] * src.z; acc.w += wc[3 * taps + j] * src.w;
    }
    st4(out + (int64_t)t * d + c, acc);
    if (wr != nullptr) {
      if (f < K) st4(wr + (int64_t)(K - 1 - f) * d + c, h0);
      if (i == 0)
        for (int e = 0; e < K - q; ++e) st4(wr + (int64_t)e * d + c, ld4(rd + (int64_t)(e + q) * d + c));
    }
  }
}

// One workgroup per token.  Wave w takes the head items w, w + nw, ...: q heads (rms norm
// with weight -> qn fp32 and LDS), k heads (rms norm with weight -> paged cache), v heads
// (unit rms -> paged cache).  Rows >= mix_from then write the mixed queries
// qmix[t - mix_from][h][c * dim + x] = sum_r ts[h][c * rep + r] * qn[c * rep + r][x].
template <typename T>
__global__ __launch_bounds__(1024) void head_norm_append_kernel(
    const T* __restrict__ qkv, int64_t stride, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int dim, int vdim, int BS,
    float* __restrict__ qn, const float* __restrict__ ts, float* __restrict__ qmix, int mix_from) {
  extern __shared__ float qs[];                        // [H * dim]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* row = qkv + (int64_t)t * stride;
  const int slot = slots[t];
  const int Lq = dim >> 3, Lv = vdim >> 3;
  const bool vec = dim % 8 == 0 && vdim % 8 == 0 && Lq <= 64 && Lv <= 64 && (Lq & (Lq - 1)) == 0 &&
                   (Lv & (Lv - 1)) == 0 && stride % 8 == 0;
  if (vec) {
    // 16-byte accesses: a head is dim / 8 (vdim / 8) lanes wide, several heads per wave pass
    {
      const int hp = 64 / Lq, sub = lane / Lq, li = lane - sub * Lq;
      for (int base = wid * hp; base < H + G; base += nw * hp) {
        const int it = base + sub;
        const bool valid = it < H + G;
        float f[8];
        ld8(row + (int64_t)(valid ? it : 0) * dim + li * 8, f);
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) ss += f[k] * f[k];
        for (int o = Lq >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float r = 1.0f / sqrtf(ss / (float)dim + eps);
        float wv[8];
        ld8((valid && it >= H) ? k_w + li * 8 : q_w + li * 8, wv);
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] = f[k] * r * wv[k];
        if (valid && it < H) {
          st8(qn + ((int64_t)t * H + it) * dim + li * 8, f);
#pragma unroll
          for (int k = 0; k < 8; ++k) qs[it * dim + li * 8 + k] = f[k];
        } else if (valid && slot >= 0) {
          st8(k_cache + (((int64_t)(slot / BS) * G + (it - H)) * BS + slot % BS) * (int64_t)dim + li * 8, f);
        }
      }
    }
    {
      const int hp = 64 / Lv, sub = lane / Lv, li = lane - sub * Lv;
      const T* vrow = row + (int64_t)(H + G) * dim;
      for (int base = wid * hp; base < G; base += nw * hp) {
        const int it = base + sub;
        const bool valid = it < G;
        float f[8];
        ld8(vrow + (int64_t)(valid ? it : 0) * vdim + li * 8, f);
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) ss += f[k] * f[k];
        for (int o = Lv >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float r = 1.0f / sqrtf(ss / (float)vdim + eps);
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] *= r;
        if (valid && slot >= 0)
          st8(v_cache + (((int64_t)(slot / BS) * G + it) * BS + slot % BS) * (int64_t)vdim + li * 8, f);
      }
    }
  } else
  for (int it = wid; it < H + 2 * G; it += nw) {
    const bool is_q = it < H, is_k = !is_q && it < H + G;
    const int n = (is_q || is_k) ? dim : vdim;
    const T* src = is_q ? row + (int64_t)it * dim
                        : is_k ? row + (int64_t)H * dim + (int64_t)(it - H) * dim
                               : row + (int64_t)(H + G) * dim + (int64_t)(it - H - G) * vdim;
    float ss = 0.f;
    for (int x = lane; x < n; x += 64) {
      const float v = ldf(src + x);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)n + eps);
    if (is_q) {
      for (int x = lane; x < n; x += 64) {
        const float v = ldf(src + x) * r * q_w[x];
        qs[it * dim + x] = v;
        qn[((int64_t)t * H + it) * dim + x] = v;
      }
    } else if (slot >= 0) {
      const int c = is_k ? it - H : it - H - G;
      T* dst = (is_k ? k_cache : v_cache) +
               (((int64_t)(slot / BS) * G + c) * BS + slot % BS) * (int64_t)n;
      for (int x = lane; x < n; x += 64)
        stf(dst + x, is_k ? ldf(src + x) * r * k_w[x] : ldf(src + x) * r);
    }
  }
  if (qmix == nullptr || t < mix_from) return;
  __syncthreads();
  const int rep = H / G, E = G * dim;
  float* om = qmix + (int64_t)(t - mix_from) * H * E;
  for (int idx = threadIdx.x; idx < H * E; idx += blockDim.x) {
    const int hh = idx / E, e = idx - hh * E, c = e / dim, x = e - c * dim;
    float a = 0.f;
    for (int r = 0; r < rep; ++r) a += ts[hh * H + c * rep + r] * qs[(c * rep + r) * dim + x];
    om[idx] = a;
  }
}

// g = min(gate, limit), u = clamp(up, -limit, limit); out = g * sigmoid(alpha g) * (u + 1).
template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_kernel(const T* __restrict__ gu, int64_t stride,
                                                          T* __restrict__ out, int64_t ostride,
                                                          int F, float limit, float alpha) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= F) return;
  const T* r = gu + (int64_t)t * stride;
  const float g = fminf(ldf(r + c), limit);
  const float u = fminf(fmaxf(ldf(r + F + c), -limit), limit);
  stf(out + (int64_t)t * ostride + c, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

// Four columns per thread (F and the row strides multiples of 4).
template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_vec_kernel(const T* __restrict__ gu,
                                                              int64_t stride, T* __restrict__ out,
                                                              int64_t ostride, int F, float limit,
                                                              float alpha) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (c >= F) return;
  const T* r = gu + (int64_t)t * stride;
  const float4 g4 = ld4(r + c), u4 = ld4(r + F + c);
  const float gs[4] = {g4.x, g4.y, g4.z, g4.w}, us[4] = {u4.x, u4.y, u4.z, u4.w};
  float o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float g = fminf(gs[k], limit);
    const float u = fminf(fmaxf(us[k], -limit), limit);
    o[k] = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
  }
  st4(out + (int64_t)t * ostride + c, make_float4(o[0], o[1], o[2], o[3]));
}

// ------------------------------------------------------------------ launchers
#define MIX_DISPATCH(f32, ...)              \
  do {                                      \
    if (f32) { typedef float T; __VA_ARGS__; } \
    else { typedef bf16_t T; __VA_ARGS__; }  \
  } while (0)

void launch_embed_sinusoid(bool f32, const int32_t* ids, const int32_t* pos, const void* table,
                           const float* inv_freq, float scale, float* out, int T_, int d, int vocab,
                           hipStream_t s) {
  if (T_ == 0) return;
  MIX_DISPATCH(f32, hipLaunchKernelGGL(embed_sinusoid_kernel<T>, dim3(T_), dim3(256), 0, s, ids, pos,
                                       (const T*)table, inv_freq, scale, out, d, vocab));
}

void launch_sandwich_norm(bool f32, const void* y, int64_t y_stride, float* residual,
                          const float* w_post, const float* gain, const float* w_pre, float* out,
                          int T_, int d, float eps, hipStream_t s) {
  if (T_ == 0) return;
  if (d % 4 == 0 && d <= 8192 && y_stride % 4 == 0) {
#define SANDWICH_VEC(n)                                                                          \
  MIX_DISPATCH(f32, hipLaunchKernelGGL((sandwich_norm_vec_kernel<T, n>), dim3(T_), dim3(256), 0, s, \
                                       (const T*)y, y_stride, residual, w_post, gain, w_pre, out, d, \
                                       eps))
    if (d <= 1024) SANDWICH_VEC(1);
    else if (d <= 2048) SANDWICH_VEC(2);
    else if (d <= 4096) SANDWICH_VEC(4);
    else SANDWICH_VEC(8);
#undef SANDWICH_VEC
    return;
  }
  MIX_DISPATCH(f32, hipLaunchKernelGGL(sandwich_norm_kernel<T>, dim3(T_), dim3(256), 0, s,
                                       (const T*)y, y_stride, residual, w_post, gain, w_pre, out, d,
                                       eps));
}

void launch_canon_conv(bool f32, const float* h, const float* w, float* state,
                       const int32_t* row_state, const int32_t* row_back, const int32_t* row_fwd,
                       const int32_t* pos, void* out, int T_, int d, int taps, int slots,
                       hipStream_t s) {
  if (T_ == 0) return;
  if (d % 4 == 0 && taps <= kVecTaps) {
#define CANON_VEC(n)                                                                              \
  MIX_DISPATCH(f32, hipLaunchKernelGGL((canon_conv_vec_kernel<T, n>), dim3(T_), dim3(256), 0, s, h, \
                                       w, state, row_state, row_back, row_fwd, pos, (T*)out, d,   \
                                       slots))
    if (taps == 1) CANON_VEC(1);
    else if (taps == 2) CANON_VEC(2);
    else if (taps == 3) CANON_VEC(3);
    else CANON_VEC(4);
#undef CANON_VEC
    return;
  }
  MIX_DISPATCH(f32, hipLaunchKernelGGL(canon_conv_kernel<T>, dim3(T_), dim3(256), 0, s, h, w, state,
                                       row_state, row_back, row_fwd, pos, (T*)out, d, taps, slots));
}

void launch_head_norm_append(bool f32, const void* qkv, int64_t stride, const float* q_w,
                             const float* k_w, float eps, const int32_t* slots, void* k_cache,
                             void* v_cache, int T_, int H, int G, int dim, int vdim, int BS,
                             float* qn, const float* ts, float* qmix, int mix_from, hipStream_t s) {
  if (T_ == 0) return;
  const size_t lds = (size_t)H * dim * sizeof(float);       // checked <= 64 KB by the caller
  const int threads = H + 2 * G >= 16 ? 1024 : 256;     // a wave per head item, up to 16 at once
  MIX_DISPATCH(f32, hipLaunchKernelGGL(head_norm_append_kernel<T>, dim3(T_), dim3(threads), lds, s,
                                       (const T*)qkv, stride, q_w, k_w, eps, slots, (T*)k_cache,
                                       (T*)v_cache, H, G, dim, vdim, BS, qn, ts, qmix, mix_from));
}

void launch_glu_clamped(bool f32, const void* gu, int64_t stride, void* out, int64_t ostride,
                        int T_, int F, float limit, float alpha, hipStream_t s) {
  if (T_ == 0) return;
  if (F % 4 == 0 && stride % 4 == 0 && ostride % 4 == 0) {
    MIX_DISPATCH(f32, hipLaunchKernelGGL(glu_clamped_vec_kernel<T>, dim3(T_, (F / 4 + 255) / 256),
                                         dim3(256), 0, s, (const T*)gu, stride, (T*)out, ostride, F,
                                         limit, alpha));
    return;
  }
  MIX_DISPATCH(f32, hipLaunchKernelGGL(glu_clamped_kernel<T>, dim3(T_, (F + 255) / 256), dim3(256),
                                       0, s, (const T*)gu, stride, (T*)out, ostride, F, limit,
                                       alpha));
}

}  // namespace rfqmix
