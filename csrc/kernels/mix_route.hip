// Mixture of experts with grouped sigmoid routing, any sizes, either activation type.
//
//   s = sigmoid(z)                       router scores (z: fp32 router logits)
//   choice = s + correction              chooses; the weights use s
//   groups: `groups` equal groups of neighbouring experts, a group's score = the sum of its two
//           largest choice scores; only experts of the `keep` best groups can be chosen
//   weights = s[chosen] / (sum + 1e-20)
//
// The expert products here are the general path: one (token, choice) pair per workgroup
// streams its expert's rows (weights stay in L2 between pairs of the same expert).  Steps of
// bf16 models whose sizes fit the grouped MFMA GEMMs use those instead.
#include "mix_common.h"

namespace rfqmix {

constexpr float kNegInfR = -__builtin_huge_valf();

// One thread per token.  Ties go to the lower index (strict comparisons, ascending scans).
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(
    const float* __restrict__ z, const float* __restrict__ corr, int T, int E, int top, int groups,
    int keep, int32_t* __restrict__ ids, float* __restrict__ weights) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* zr = z + (int64_t)t * E;
  int32_t* id = ids + (int64_t)t * top;
  float* wt = weights + (int64_t)t * top;
  uint64_t kept = ~0ull;
  int per = E;
  if (groups > 0) {
    per = E / groups;
    kept = 0;
    for (int a = 0; a < keep; ++a) {
      int best = -1;
      float bs = 0.f;
      for (int g = 0; g < groups; ++g) {
        if ((kept >> g) & 1) continue;
        float m1 = kNegInfR, m2 = kNegInfR;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float c = 1.0f / (1.0f + expf(-zr[e])) + corr[e];
          if (c > m1) { m2 = m1; m1 = c; } else if (c > m2) { m2 = c; }
        }
        const float sc = per > 1 ? m1 + m2 : m1;
        if (best < 0 || sc > bs) { best = g; bs = sc; }
      }
      kept |= 1ull << best;
    }
  }
  float sum = 0.f;
  for (int a = 0; a < top; ++a) {
    int best = -1;
    float bc = 0.f, bsc = 0.f;
    for (int e = 0; e < E; ++e) {
      if (groups > 0 && !((kept >> (e / per)) & 1)) continue;
      bool used = false;
      for (int b = 0; b < a; ++b) used |= id[b] == e;
      if (used) continue;
      const float s = 1.0f / (1.0f + expf(-zr[e]));
      const float c = s + corr[e];
      if (best < 0 || c > bc) { best = e; bc = c; bsc = s; }
    }
    id[a] = best;
    wt[a] = bsc;
    sum += bsc;
  }
  const float inv = 1.0f / (sum + 1e-20f);
  for (int a = 0; a < top; ++a) wt[a] *= inv;
}

// act[p, f] = silu(Wg[e] . x_t) * (Wu[e] . x_t) for pair p = t * top + k, e = ids[p].
// Grid (pairs, feature tiles of FT); x_t staged in LDS as floats; one wave per feature.
template <typename T>
__global__ __launch_bounds__(256) void moe_pair_up_kernel(
    const T* __restrict__ h, int64_t h_stride, const int32_t* __restrict__ ids,
    const T* __restrict__ w13, T* __restrict__ act, int top, int d, int F, int E, int FT) {
  extern __shared__ float xs[];
  const int p = blockIdx.x, t = p / top;
  const int e = ids[p];
  if (e < 0 || e >= E) return;
  for (int c = threadIdx.x; c < d; c += blockDim.x) xs[c] = ldf(h + (int64_t)t * h_stride + c);
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* wg = w13 + (int64_t)e * 2 * F * d;
  const int f1 = min(F, (blockIdx.y + 1) * FT);
  for (int f = blockIdx.y * FT + wid; f < f1; f += nw) {
    const T* g = wg + (int64_t)f * d;
    const T* u = wg + (int64_t)(F + f) * d;
    float ag = 0.f, au = 0.f;
    for (int c = lane; c < d; c += 64) {
      const float x = xs[c];
      ag += ldf(g + c) * x;
      au += ldf(u + c) * x;
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) stf(act + (int64_t)p * F + f, ag / (1.0f + expf(-ag)) * au);
  }
}

// out[t, c] = base[t, c] + sum_k weights[t, k] * (W2[ids[t, k]][c, :] . act[t * top + k, :]).
// Grid (tokens, column tiles of CT); the token's `top` activation rows staged in LDS.
template <typename T>
__global__ __launch_bounds__(256) void moe_pair_down_kernel(
    const T* __restrict__ act, const int32_t* __restrict__ ids, const float* __restrict__ weights,
    const T* __restrict__ w2, const T* __restrict__ base, int64_t base_stride,
    float* __restrict__ out, int top, int d, int F, int E, int CT) {
  extern __shared__ float as[];                // [top][F]
  const int t = blockIdx.x;
  for (int x = threadIdx.x; x < top * F; x += blockDim.x)
    as[x] = ldf(act + (int64_t)t * top * F + x);
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int c1 = min(d, (blockIdx.y + 1) * CT);
  for (int c = blockIdx.y * CT + wid; c < c1; c += nw) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[(int64_t)t * top + k];
      if (e < 0 || e >= E) continue;
      const T* row = w2 + ((int64_t)e * d + c) * F;
      const float* a = as + k * F;
      float dot = 0.f;
      for (int f = lane; f < F; f += 64) dot += ldf(row + f) * a[f];
      acc += weights[(int64_t)t * top + k] * dot;
    }
    acc = wave_sum(acc);
    if (lane == 0)
      out[(int64_t)t * d + c] = acc + (base != nullptr ? ldf(base + (int64_t)t * base_stride + c) : 0.f);
  }
}

// ------------------------------------------------------------------ launchers
void launch_moe_route_grouped(const float* z, const float* corr, int T, int E, int top, int groups,
                              int keep, int32_t* ids, float* weights, hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((T + 255) / 256), dim3(256), 0, s, z, corr, T,
                     E, top, groups, keep, ids, weights);
}

void launch_moe_pair_up(bool f32, const void* h, int64_t h_stride, const int32_t* ids,
                        const void* w13, void* act, int pairs, int top, int d, int F, int E,
                        hipStream_t s) {
  if (pairs == 0) return;
  const int FT = 64;
  const dim3 grid(pairs, (F + FT - 1) / FT);
  const size_t lds = (size_t)d * 4;
  if (f32)
    hipLaunchKernelGGL(moe_pair_up_kernel<float>, grid, dim3(256), lds, s, (const float*)h,
                       h_stride, ids, (const float*)w13, (float*)act, top, d, F, E, FT);
  else
    hipLaunchKernelGGL(moe_pair_up_kernel<bf16_t>, grid, dim3(256), lds, s, (const bf16_t*)h,
                       h_stride, ids, (const bf16_t*)w13, (bf16_t*)act, top, d, F, E, FT);
}

void launch_moe_pair_down(bool f32, const void* act, const int32_t* ids, const float* weights,
                          const void* w2, const void* base, int64_t base_stride, float* out, int T,
                          int top, int d, int F, int E, hipStream_t s) {
  if (T == 0) return;
  const int CT = 64;
  const dim3 grid(T, (d + CT - 1) / CT);
  const size_t lds = (size_t)top * F * 4;
  static bool attr = false;
  if (!attr) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_pair_down_kernel<float>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_pair_down_kernel<bf16_t>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  if (f32)
    hipLaunchKernelGGL(moe_pair_down_kernel<float>, grid, dim3(256), lds, s, (const float*)act, ids,
                       weights, (const float*)w2, (const float*)base, base_stride, out, top, d, F,
                       E, CT);
  else
    hipLaunchKernelGGL(moe_pair_down_kernel<bf16_t>, grid, dim3(256), lds, s, (const bf16_t*)act,
                       ids, weights, (const bf16_t*)w2, (const bf16_t*)base, base_stride, out, top,
                       d, F, E, CT);
}

}  // namespace rfqmix
