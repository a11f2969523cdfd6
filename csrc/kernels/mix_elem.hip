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
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float ang = p * inv_freq[c >> 1];
    const float pe = (c & 1) ? cosf(ang) : sinf(ang);
    o[c] = ldf(row + c) * scale + pe;
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

// One workgroup per token.  Wave w takes the head items w, w + nw, ...: q heads (rms norm
// with weight -> qn fp32 and LDS), k heads (rms norm with weight -> paged cache), v heads
// (unit rms -> paged cache).  Rows >= mix_from then write the mixed queries
// qmix[t - mix_from][h][c * dim + x] = sum_r ts[h][c * rep + r] * qn[c * rep + r][x].
template <typename T>
__global__ __launch_bounds__(256) void head_norm_append_kernel(
    const T* __restrict__ qkv, int64_t stride, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int dim, int vdim, int BS,
    float* __restrict__ qn, const float* __restrict__ ts, float* __restrict__ qmix, int mix_from) {
  extern __shared__ float qs[];                        // [H * dim]
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* row = qkv + (int64_t)t * stride;
  const int slot = slots[t];
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
  MIX_DISPATCH(f32, hipLaunchKernelGGL(sandwich_norm_kernel<T>, dim3(T_), dim3(256), 0, s,
                                       (const T*)y, y_stride, residual, w_post, gain, w_pre, out, d,
                                       eps));
}

void launch_canon_conv(bool f32, const float* h, const float* w, float* state,
                       const int32_t* row_state, const int32_t* row_back, const int32_t* row_fwd,
                       const int32_t* pos, void* out, int T_, int d, int taps, int slots,
                       hipStream_t s) {
  if (T_ == 0) return;
  MIX_DISPATCH(f32, hipLaunchKernelGGL(canon_conv_kernel<T>, dim3(T_), dim3(256), 0, s, h, w, state,
                                       row_state, row_back, row_fwd, pos, (T*)out, d, taps, slots));
}

void launch_head_norm_append(bool f32, const void* qkv, int64_t stride, const float* q_w,
                             const float* k_w, float eps, const int32_t* slots, void* k_cache,
                             void* v_cache, int T_, int H, int G, int dim, int vdim, int BS,
                             float* qn, const float* ts, float* qmix, int mix_from, hipStream_t s) {
  if (T_ == 0) return;
  const size_t lds = (size_t)H * dim * sizeof(float);       // checked <= 64 KB by the caller
  MIX_DISPATCH(f32, hipLaunchKernelGGL(head_norm_append_kernel<T>, dim3(T_), dim3(256), lds, s,
                                       (const T*)qkv, stride, q_w, k_w, eps, slots, (T*)k_cache,
                                       (T*)v_cache, H, G, dim, vdim, BS, qn, ts, qmix, mix_from));
}

void launch_glu_clamped(bool f32, const void* gu, int64_t stride, void* out, int64_t ostride,
                        int T_, int F, float limit, float alpha, hipStream_t s) {
  if (T_ == 0) return;
  MIX_DISPATCH(f32, hipLaunchKernelGGL(glu_clamped_kernel<T>, dim3(T_, (F + 255) / 256), dim3(256),
                                       0, s, (const T*)gu, stride, (T*)out, ostride, F, limit,
                                       alpha));
}

}  // namespace rfqmix
