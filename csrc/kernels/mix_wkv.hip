// The wkv recurrent mixer: token-shift mixes of a layer's input and the per-head recurrence
//
//   w_t = exp(-exp(zw_t + w0))                       decay per key channel, fp32
//   o_t = (S + diag(u) k_t v_t^T)^T r_t              the bonus u counts for the current token only
//   S  <- diag(w_t) S + k_t v_t^T                    S: N key x N value channels, fp32
//   out_t = o_t / rms_head(o_t) * norm_w * silu(gate_t)
//
// Rows of a sequence are contiguous in a step (a "run").  row_state = slot * 2 + half to read
// (-1: none), row_back = index of the row inside its run, row_fwd = rows of the run after it.
// State pools are double buffered: a run reads its sequence's half and writes the other, and
// a run that starts at position 0 reads nothing (the slot may hold another sequence's rest).
#include "mix_common.h"

namespace rfqmix {

// out[s, t, :] = x[t] + (x'[t] - x[t]) * mu[s]; x' = previous token's row.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(
    const float* __restrict__ x, const float* __restrict__ mu, float* __restrict__ prev,
    const int32_t* __restrict__ row_state, const int32_t* __restrict__ row_back,
    const int32_t* __restrict__ row_fwd, const int32_t* __restrict__ pos, T* __restrict__ out,
    int Trows, int d, int NS, int slots) {
  const int t = blockIdx.x;
  const int code = row_state[t], i = row_back[t], f = row_fwd[t], p = pos[t];
  const float* xr = x + (int64_t)t * d;
  const float* before = nullptr;
  if (i > 0)
    before = xr - d;
  else if (p > 0 && code >= 0)
    before = prev + ((int64_t)(code & 1) * slots + (code >> 1)) * d;
  float* keep = (f == 0 && code >= 0)
                    ? prev + ((int64_t)(1 - (code & 1)) * slots + (code >> 1)) * d
                    : nullptr;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float a = xr[c];
    const float b = before != nullptr ? before[c] : 0.f;
    if (keep != nullptr) keep[c] = a;
    for (int s = 0; s < NS; ++s)
      stf(out + ((int64_t)s * Trows + t) * d + c, a + (b - a) * mu[(int64_t)s * d + c]);
  }
}

// One workgroup per (row, head); only a run's first row works: it walks the run token by
// token.  Thread j owns value channel j: column j of S lives in LDS (st[i * N + j]: lanes hit
// consecutive banks), or in registers when N is the compile-time NR.  r, k and the decay of
// the next token are fetched while the current one is computed.
template <typename T, int NR>
__global__ __launch_bounds__(256) void wkv_recurrence_kernel(
    const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ zw, const T* __restrict__ gate, int64_t r_stride, int64_t k_stride,
    int64_t v_stride, int64_t zw_stride, int64_t g_stride, const float* __restrict__ w0,
    const float* __restrict__ u, const float* __restrict__ norm_w, float eps,
    float* __restrict__ state, const int32_t* __restrict__ row_state,
    const int32_t* __restrict__ row_back, const int32_t* __restrict__ row_fwd,
    const int32_t* __restrict__ pos, const int32_t* __restrict__ run_rows, T* __restrict__ out,
    int H, int N, int slots) {
  // with a list of the runs' first rows the grid holds only workgroups that work (-1: no run);
  // without one, a workgroup per row, of which the runs' first rows work
  const int t0 = run_rows != nullptr ? run_rows[blockIdx.x] : (int)blockIdx.x;
  const int h = blockIdx.y;
  if (t0 < 0 || row_back[t0] != 0) return;
  const int n = row_fwd[t0] + 1;
  const int code = row_state[t0];
  const int j = threadIdx.x;
  const bool live = j < N;
  const int ch = h * N + (live ? j : 0);

  extern __shared__ __attribute__((aligned(16))) float lds[];
  // [2][N] of (r, k, decay, bonus) by key channel for the current / next token: one 16-byte
  // LDS read per channel in the sum below
  float4* rk = reinterpret_cast<float4*>(lds);
  float* scratch = lds + 8 * N;      // 16
  float* st = scratch + 16;          // [N][N] when NR == 0
  float sreg[NR > 0 ? NR : 1];

  const bool from_state = code >= 0 && pos[t0] > 0;
  const float* rd = state + (((int64_t)(code & 1) * slots + (code >> 1)) * H + h) * (int64_t)N * N;
  if (NR > 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i) sreg[i] = (from_state && live) ? rd[i * N + j] : 0.f;
  } else {
    if (live)
      for (int i = 0; i < N; ++i) st[i * N + j] = from_state ? rd[i * N + j] : 0.f;
  }

  float nr = 0.f, nk = 0.f, nw = 0.f, nv = 0.f, ng = 0.f;
  if (live) {
    nr = ldf(r + (int64_t)t0 * r_stride + ch);
    nk = ldf(k + (int64_t)t0 * k_stride + ch);
    nw = expf(-expf(ldf(zw + (int64_t)t0 * zw_stride + ch) + w0[ch]));
    nv = ldf(v + (int64_t)t0 * v_stride + ch);
    ng = ldf(gate + (int64_t)t0 * g_stride + ch);
  }
  const float my_nw = live ? norm_w[ch] : 0.f;
  const float my_u = live ? u[ch] : 0.f;

  for (int a = 0; a < n; ++a) {
    const float4* cur = rk + (a & 1) * N;
    if (live) rk[(a & 1) * N + j] = make_float4(nr, nk, nw, my_u);
    const float vj = nv, gj = ng;
    __syncthreads();
    if (a + 1 < n && live) {           // the next token's operands, in flight during the sums
      const int64_t t = t0 + a + 1;
      nr = ldf(r + t * r_stride + ch);
      nk = ldf(k + t * k_stride + ch);
      nw = ldf(zw + t * zw_stride + ch);
      nv = ldf(v + t * v_stride + ch);
      ng = ldf(gate + t * g_stride + ch);
    }
    float o = 0.f;
    if (live) {
      if (NR > 0) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const float4 c4 = cur[i];
          const float kv = c4.y * vj;
          o += c4.x * (sreg[i] + c4.w * kv);
          sreg[i] = c4.z * sreg[i] + kv;
        }
      } else {
        for (int i = 0; i < N; ++i) {
          const float4 c4 = cur[i];
          const float s = st[i * N + j];
          const float kv = c4.y * vj;
          o += c4.x * (s + c4.w * kv);
          st[i * N + j] = c4.z * s + kv;
        }
      }
    }
    if (a + 1 < n && live) nw = expf(-expf(nw + w0[ch]));
    const float ss = block_sum(live ? o * o : 0.f, scratch);
    if (live) {
      const float y = o / sqrtf(ss / (float)N + eps) * my_nw * (gj / (1.0f + expf(-gj)));
      stf(out + (int64_t)(t0 + a) * H * N + ch, y);
    }
  }
  if (code >= 0 && live) {
    float* wr = state + (((int64_t)(1 - (code & 1)) * slots + (code >> 1)) * H + h) * (int64_t)N * N;
    if (NR > 0) {
#pragma unroll
      for (int i = 0; i < NR; ++i) wr[i * N + j] = sreg[i];
    } else {
      for (int i = 0; i < N; ++i) wr[i * N + j] = st[i * N + j];
    }
  }
}

// ------------------------------------------------------------------ launchers
void launch_token_shift_mix(bool out_f32, const float* x, const float* mu, float* prev,
                            const int32_t* row_state, const int32_t* row_back,
                            const int32_t* row_fwd, const int32_t* pos, void* out, int T, int d,
                            int NS, int slots, hipStream_t s) {
  if (T == 0) return;
  if (out_f32)
    hipLaunchKernelGGL(token_shift_mix_kernel<float>, dim3(T), dim3(256), 0, s, x, mu, prev,
                       row_state, row_back, row_fwd, pos, (float*)out, T, d, NS, slots);
  else
    hipLaunchKernelGGL(token_shift_mix_kernel<bf16_t>, dim3(T), dim3(256), 0, s, x, mu, prev,
                       row_state, row_back, row_fwd, pos, (bf16_t*)out, T, d, NS, slots);
}

template <typename T, int NR>
static void launch_wkv_one(const void* r, const void* k, const void* v, const void* zw,
                           const void* gate, int64_t rs, int64_t ks, int64_t vs, int64_t zs,
                           int64_t gs, const float* w0, const float* u, const float* norm_w,
                           float eps, float* state, const int32_t* row_state,
                           const int32_t* row_back, const int32_t* row_fwd, const int32_t* pos,
                           const int32_t* run_rows, int runs, void* out, int Trows, int H, int N,
                           int slots, hipStream_t s) {
  const int threads = (N + 63) / 64 * 64;
  const size_t lds = (size_t)(8 * N + 16 + (NR > 0 ? 0 : N * N)) * 4;
  static bool attr = false;
  if (!attr) {          // dynamic LDS above 64 KB has to be allowed per kernel, once
    hipFuncSetAttribute(reinterpret_cast<const void*>(&wkv_recurrence_kernel<T, NR>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  hipLaunchKernelGGL((wkv_recurrence_kernel<T, NR>), dim3(run_rows != nullptr ? runs : Trows, H),
                     dim3(threads), lds, s, (const T*)r, (const T*)k, (const T*)v, (const T*)zw,
                     (const T*)gate, rs, ks, vs, zs, gs, w0, u, norm_w, eps, state, row_state,
                     row_back, row_fwd, pos, run_rows, (T*)out, H, N, slots);
}

// Whether the head size fits (threads <= 256; the state matrix of a head in LDS).
bool wkv_ok(int N) { return N >= 1 && N <= 192; }

void launch_wkv_recurrence(bool f32, const void* r, const void* k, const void* v, const void* zw,
                           const void* gate, int64_t rs, int64_t ks, int64_t vs, int64_t zs,
                           int64_t gs, const float* w0, const float* u, const float* norm_w,
                           float eps, float* state, const int32_t* row_state,
                           const int32_t* row_back, const int32_t* row_fwd, const int32_t* pos,
                           const int32_t* run_rows, int runs, void* out, int Trows, int H, int N,
                           int slots, hipStream_t s) {
  if (Trows == 0 || (run_rows != nullptr && runs == 0)) return;
#define WKV_GO(TT, NRR)                                                                         \
  launch_wkv_one<TT, NRR>(r, k, v, zw, gate, rs, ks, vs, zs, gs, w0, u, norm_w, eps, state,     \
                          row_state, row_back, row_fwd, pos, run_rows, runs, out, Trows, H, N,  \
                          slots, s)
  if (f32) {
    if (N == 64) WKV_GO(float, 64); else WKV_GO(float, 0);
  } else {
    if (N == 64) WKV_GO(bf16_t, 64); else WKV_GO(bf16_t, 0);
  }
#undef WKV_GO
}

}  // namespace rfqmix
