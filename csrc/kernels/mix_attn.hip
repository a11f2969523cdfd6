// Paged attention of the layer-list models: per-head distance bias, scores mixed over heads,
// block ("chunk") causal mask, softmax with a per-head sink logit in the denominator.
//
//   score_g(i, j)  = scale q_g(i).k_{kv(g)}(j) - slope_g (i - j)
//   score'_h(i, j) = sum_g talk[h, g] score_g(i, j)
//   i sees j <= i with floor(i / chunk) = floor(j / chunk)   (chunk = 0: plain causal)
//   w_h(i, j) = exp(score'_h) / (exp(sink_h) + sum_j' exp(score'_h(i, j')))
//
// The sink has no key and no value: it is the initial state (m = sink, l = 1, o = 0) of the
// online softmax.
//
// Two kernels, any head count and head sizes (fp32 FMA; scores and softmax in fp32):
//   attn_talk_decode    one workgroup per token row of a decode / short-extend sequence,
//                       every head in the workgroup: raw scores of a key tile for all heads
//                       in LDS, mixed there (H^2 per key), softmax and P.V per head.
//   attn_mixq_prefill   one workgroup per (sequence, query block, head) on pre-mixed
//                       queries: the mixing is linear in q, so head h's mixed score is the
//                       product of q~[h] (G * dim wide, one part per key/value head) with the
//                       concatenated key heads; slopes arrive mixed.  MFMA tiles for bf16
//                       models whose sizes fit them are in mix_attn_mfma.hip.
#include "mix_common.h"

namespace rfqmix {

constexpr float kNegInf = -__builtin_huge_valf();

// ------------------------------------------------------------------ decode rows
// LDS (floats): qs[H*dim] | kt[KT*(dim+1)] | sc[H*KT] | sm[H*KT] | tk[H*H] | acc[H*vdim] |
//               mrow[H] | lrow[H] | arow[H]
template <typename T>
__global__ __launch_bounds__(256) void attn_talk_decode_kernel(
    const float* __restrict__ qn, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int maxb, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len, T* __restrict__ out,
    int64_t out_stride, const float* __restrict__ slopes, const float* __restrict__ talk,
    const float* __restrict__ sink, float scale, int chunk, int H, int G, int dim, int vdim,
    int BS, int KT) {
  const int s = blockIdx.x, r = blockIdx.y;
  const int ql = q_len[s];
  if (r >= ql) return;
  const int t = q_start[s] + r;
  const int p = kv_len[s] - ql + r;                    // position of this row
  const int j0 = chunk > 0 ? (p / chunk) * chunk : 0;
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int rep = H / G;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, nw = blockDim.x >> 6;
  const int nthr = blockDim.x;

  extern __shared__ float lds[];
  float* qs = lds;
  float* kt = qs + H * dim;
  float* sc = kt + KT * (dim + 1);
  float* sm = sc + H * KT;
  float* tk = sm + H * KT;
  float* acc = tk + H * H;
  float* mrow = acc + H * vdim;
  float* lrow = mrow + H;
  float* arow = lrow + H;

  for (int x = tid; x < H * dim; x += nthr) qs[x] = qn[(int64_t)t * H * dim + x];
  if (talk != nullptr)
    for (int x = tid; x < H * H; x += nthr) tk[x] = talk[x];
  for (int x = tid; x < H * vdim; x += nthr) acc[x] = 0.f;
  for (int x = tid; x < H; x += nthr) {
    mrow[x] = sink != nullptr ? sink[x] : kNegInf;
    lrow[x] = sink != nullptr ? 1.f : 0.f;
  }
  __syncthreads();

  for (int jb = j0; jb <= p; jb += KT) {
    const int nk = min(KT, p + 1 - jb);
    // (1) raw scores, one key/value head at a time through LDS
    for (int c = 0; c < G; ++c) {
      for (int x = tid; x < nk * dim; x += nthr) {
        const int jj = x / dim, e = x - jj * dim, j = jb + jj;
        const T* kr = k_cache + (((int64_t)bt[j / BS] * G + c) * BS + j % BS) * (int64_t)dim;
        kt[jj * (dim + 1) + e] = ldf(kr + e);
      }
      __syncthreads();
      for (int x = tid; x < rep * KT; x += nthr) {
        const int rr = x / KT, jj = x - rr * KT, g = c * rep + rr;
        float a = kNegInf;
        if (jj < nk) {
          const float* qv = qs + g * dim;
          const float* kv = kt + jj * (dim + 1);
          float d0 = 0.f;
          for (int e = 0; e < dim; ++e) d0 += qv[e] * kv[e];
          a = d0 * scale - slopes[g] * (float)(p - (jb + jj));
        }
        sc[g * KT + jj] = a;
      }
      __syncthreads();
    }
    // (2) mix over heads (keys past the tile's end stay -inf)
    for (int x = tid; x < H * KT; x += nthr) {
      const int hh = x / KT, jj = x - hh * KT;
      float a = kNegInf;
      if (jj < nk) {
        if (talk != nullptr) {
          a = 0.f;
          for (int g = 0; g < H; ++g) a += tk[hh * H + g] * sc[g * KT + jj];
        } else {
          a = sc[x];
        }
      }
      sm[x] = a;
    }
    __syncthreads();
    // (3) online softmax, one wave per head
    for (int hh = wid; hh < H; hh += nw) {
      float mx = kNegInf;
      for (int jj = lane; jj < KT; jj += 64) mx = fmaxf(mx, sm[hh * KT + jj]);
      mx = wave_max(mx);
      const float mo = mrow[hh];
      const float mn = fmaxf(mo, mx);
      float sum = 0.f;
      for (int jj = lane; jj < KT; jj += 64) {
        const float v = sm[hh * KT + jj];
        const float e = v == kNegInf ? 0.f : expf(v - mn);
        sm[hh * KT + jj] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float al = mo == kNegInf ? 0.f : expf(mo - mn);
        arow[hh] = al;
        lrow[hh] = lrow[hh] * al + sum;
        mrow[hh] = mn;
      }
    }
    __syncthreads();
    // (4) acc[h] = acc[h] * alpha + P[h] . V[kv(h)]
    for (int x = tid; x < H * vdim; x += nthr) {
      const int hh = x / vdim, dv = x - hh * vdim, c = hh / rep;
      float a = acc[x] * arow[hh];
      for (int jj = 0; jj < nk; ++jj) {
        const int j = jb + jj;
        const T* vr = v_cache + (((int64_t)bt[j / BS] * G + c) * BS + j % BS) * (int64_t)vdim;
        a += sm[hh * KT + jj] * ldf(vr + dv);
      }
      acc[x] = a;
    }
    __syncthreads();
  }
  T* o = out + (int64_t)t * out_stride;
  for (int x = tid; x < H * vdim; x += nthr) {
    const float l = lrow[x / vdim];
    stf(o + x, l > 0.f ? acc[x] / l : 0.f);
  }
}

// ------------------------------------------------------------------ prefill rows
// Work item (work_seq[w], work_qblk[w]) x head h; QB = 32 queries, KT = 64 keys, the G*dim
// wide product staged through LDS in slices of EC = 64.
// LDS (floats): Qs[QB][EC+1] | Ks[KT][EC+1] | Ps[QB][KT+1] | Os[QB*vdim] | al[QB] | ll[QB]
constexpr int QB = 32, KT2 = 64, EC = 64;

template <typename T>
__global__ __launch_bounds__(256) void attn_mixq_prefill_kernel(
    const float* __restrict__ qmix, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int maxb, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len,
    const int32_t* __restrict__ work_seq, const int32_t* __restrict__ work_qblk,
    T* __restrict__ out, int64_t out_stride, const float* __restrict__ slopes,
    const float* __restrict__ sink, int chunk, int H, int G, int dim, int vdim, int BS) {
  const int s = work_seq[blockIdx.x];
  if (s < 0) return;
  const int hh = blockIdx.y;
  const int qb = work_qblk[blockIdx.x];
  const int ql = q_len[s], kl = kv_len[s];
  const int i0 = qb * QB;
  if (i0 >= ql) return;
  const int nq = min(QB, ql - i0);
  const int p0 = kl - ql + i0;                         // position of the block's first query
  const int plast = p0 + nq - 1;
  const int jlo = chunk > 0 ? (p0 / chunk) * chunk : 0;
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int rep = H / G, E = G * dim, c_v = hh / rep;
  const int tid = threadIdx.x;
  const int ti = tid >> 4, tj = tid & 15;              // rows ti, ti+16; cols tj + 16k
  const float slope = slopes[hh];

  extern __shared__ float lds[];
  float* Qs = lds;
  float* Ks = Qs + QB * (EC + 1);
  float* Ps = Ks + KT2 * (EC + 1);
  float* Os = Ps + QB * (KT2 + 1);
  float* al = Os + QB * vdim;
  float* ll = al + QB;

  for (int x = tid; x < QB * vdim; x += 256) Os[x] = 0.f;
  float m[2], l[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    m[a] = sink != nullptr ? sink[hh] : kNegInf;
    l[a] = sink != nullptr ? 1.f : 0.f;
  }
  const float* qbase = qmix + ((int64_t)(q_start[s] + i0) * H + hh) * E;

  for (int jb = jlo; jb <= plast; jb += KT2) {
    const int nk = min(KT2, plast + 1 - jb);
    float sacc[2][4] = {};
    for (int e0 = 0; e0 < E; e0 += EC) {
      const int ne = min(EC, E - e0);
      __syncthreads();
      for (int x = tid; x < QB * EC; x += 256) {
        const int i = x / EC, e = x - i * EC;
        Qs[i * (EC + 1) + e] = (i < nq && e < ne) ? qbase[(int64_t)i * H * E + e0 + e] : 0.f;
      }
      for (int x = tid; x < KT2 * EC; x += 256) {
        const int jj = x / EC, e = x - jj * EC;
        float v = 0.f;
        if (jj < nk && e < ne) {
          const int j = jb + jj, ee = e0 + e, c = ee / dim, xx = ee - c * dim;
          v = ldf(k_cache + (((int64_t)bt[j / BS] * G + c) * BS + j % BS) * (int64_t)dim + xx);
        }
        Ks[jj * (EC + 1) + e] = v;
      }
      __syncthreads();
      for (int e = 0; e < EC; ++e) {
        const float q0 = Qs[ti * (EC + 1) + e], q1 = Qs[(ti + 16) * (EC + 1) + e];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float kv = Ks[(tj + 16 * k) * (EC + 1) + e];
          sacc[0][k] += q0 * kv;
          sacc[1][k] += q1 * kv;
        }
      }
    }
    // bias, mask, online softmax; a row's 64 columns live in the 16 lanes of its group
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int i = ti + 16 * a, pi = p0 + i;
      const int klo = chunk > 0 ? (pi / chunk) * chunk : 0;   // first key of the query's block
      float mx = kNegInf;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int j = jb + tj + 16 * k;
        const bool ok = i < nq && j <= pi && j >= klo;
        sacc[a][k] = ok ? sacc[a][k] - slope * (float)(pi - j) : kNegInf;
        mx = fmaxf(mx, sacc[a][k]);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float mn = fmaxf(m[a], mx);
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float e = sacc[a][k] == kNegInf ? 0.f : expf(sacc[a][k] - mn);
        Ps[i * (KT2 + 1) + tj + 16 * k] = e;
        sum += e;
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
      const float alpha = m[a] == kNegInf ? 0.f : expf(m[a] - mn);
      l[a] = l[a] * alpha + sum;
      m[a] = mn;
      if (tj == 0) al[i] = alpha;
    }
    __syncthreads();
    for (int x = tid; x < nq * vdim; x += 256) {
      const int i = x / vdim, dv = x - i * vdim;
      float a = Os[x] * al[i];
      const float* pr = Ps + i * (KT2 + 1);
      for (int jj = 0; jj < nk; ++jj) {
        const int j = jb + jj;
        a += pr[jj] * ldf(v_cache + (((int64_t)bt[j / BS] * G + c_v) * BS + j % BS) * (int64_t)vdim + dv);
      }
      Os[x] = a;
    }
  }
  if (tj == 0) {
    ll[ti] = l[0];
    ll[ti + 16] = l[1];
  }
  __syncthreads();
  for (int x = tid; x < nq * vdim; x += 256) {
    const int i = x / vdim, dv = x - i * vdim;
    const float lv = ll[i];
    stf(out + (int64_t)(q_start[s] + i0 + i) * out_stride + (int64_t)hh * vdim + dv,
        lv > 0.f ? Os[x] / lv : 0.f);
  }
}

// ------------------------------------------------------------------ launchers
constexpr int kMaxLds = 160 * 1024;        // LDS of a gfx950 compute unit

size_t decode_lds_floats(int H, int dim, int vdim, int KT) {
  return (size_t)H * dim + (size_t)KT * (dim + 1) + 2 * (size_t)H * KT + (size_t)H * H +
         (size_t)H * vdim + 3 * (size_t)H;
}

// Returns the key tile the launch uses (0: the sizes do not fit the LDS).
int launch_attn_talk_decode(bool f32, const float* qn, const void* k_cache, const void* v_cache,
                            const int32_t* bt, int maxb, const int32_t* q_start,
                            const int32_t* q_len, const int32_t* kv_len, void* out,
                            int64_t out_stride, const float* slopes, const float* talk,
                            const float* sink, float scale, int chunk, int NA, int max_rows, int H,
                            int G, int dim, int vdim, int BS, hipStream_t s) {
  // the largest key tile whose LDS fits two workgroups per CU, else one (160 KB per CU)
  int KT = 64;
  while (KT >= 8 && decode_lds_floats(H, dim, vdim, KT) * 4 > 80 * 1024) KT >>= 1;
  if (KT < 8) {
    KT = 64;
    while (KT >= 8 && decode_lds_floats(H, dim, vdim, KT) * 4 > kMaxLds) KT >>= 1;
  }
  if (KT < 8) return 0;
  if (NA == 0) return KT;
  const size_t lds = decode_lds_floats(H, dim, vdim, KT) * 4;
  static bool attr = false;
  if (!attr) {          // dynamic LDS above 64 KB has to be allowed per kernel, once
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_talk_decode_kernel<float>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_talk_decode_kernel<bf16_t>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    attr = true;
  }
  if (f32)
    hipLaunchKernelGGL(attn_talk_decode_kernel<float>, dim3(NA, max_rows), dim3(256), lds, s, qn,
                       (const float*)k_cache, (const float*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, (float*)out, out_stride, slopes, talk, sink, scale, chunk, H, G, dim,
                       vdim, BS, KT);
  else
    hipLaunchKernelGGL(attn_talk_decode_kernel<bf16_t>, dim3(NA, max_rows), dim3(256), lds, s, qn,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, (bf16_t*)out, out_stride, slopes, talk, sink, scale, chunk, H, G,
                       dim, vdim, BS, KT);
  return KT;
}

bool launch_attn_mixq_prefill(bool f32, const float* qmix, const void* k_cache,
                              const void* v_cache, const int32_t* bt, int maxb,
                              const int32_t* q_start, const int32_t* q_len, const int32_t* kv_len,
                              const int32_t* work_seq, const int32_t* work_qblk, int W, void* out,
                              int64_t out_stride, const float* slopes, const float* sink, int chunk,
                              int H, int G, int dim, int vdim, int BS, hipStream_t s) {
  const size_t lds = ((size_t)QB * (EC + 1) + (size_t)KT2 * (EC + 1) + (size_t)QB * (KT2 + 1) +
                      (size_t)QB * vdim + 2 * QB) * 4;
  if (lds > (size_t)kMaxLds) return false;
  if (W == 0) return true;
  static bool attr = false;
  if (!attr) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mixq_prefill_kernel<float>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mixq_prefill_kernel<bf16_t>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    attr = true;
  }
  if (f32)
    hipLaunchKernelGGL(attn_mixq_prefill_kernel<float>, dim3(W, H), dim3(256), lds, s, qmix,
                       (const float*)k_cache, (const float*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, (float*)out, out_stride, slopes, sink, chunk, H,
                       G, dim, vdim, BS);
  else
    hipLaunchKernelGGL(attn_mixq_prefill_kernel<bf16_t>, dim3(W, H), dim3(256), lds, s, qmix,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, (bf16_t*)out, out_stride, slopes, sink, chunk,
                       H, G, dim, vdim, BS);
  return true;
}

}  // namespace rfqmix
