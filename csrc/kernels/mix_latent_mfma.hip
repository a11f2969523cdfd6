// MFMA latent attention for bf16 caches: multi-query attention whose single key/value head is
// the cached latent itself.
//
//   score_h(i, j) = scale q'_h(i) . c(j)            q' = the query carried into the latent space
//   w_h(i, j)     = exp(score) / (exp(sink_h) + sum_j' exp(score_h(i, j')))      j <= i
//   o'_h(i)       = sum_j w_h(i, j) c(j)            the same rows c are keys and values
//
// Tile structure of mix_attn_mfma.hip: a work item is (sequence, block of 32 query tokens); its
// columns are the (token, head) pairs, 16 per wave, 64 per workgroup, and all workgroups of a
// work item stream the same 32-token pages:
//
//   per page, staged ONCE in LDS for both products:
//     S^T[key, col]  = C[key, :] . Q'[col, :]         v_mfma_f32_16x16x32_bf16, A = latent rows
//     online softmax per column in fp32 (the sink is its initial state)
//     O^T[r, col]   += C^T[r, key] . P^T[key, col]    A = C^T by transposed LDS reads of the same
//                                                     tile, P as bf16 hi + lo parts so that the
//                                                     weights keep fp32's precision
//
// R = 32 EK wide latents (EK in 2, 4, 8, 16), any head count, 32-token pages.  Rows in LDS are
// padded by 16 B so that the rows of a fragment read fall into different banks.
#include "common.h"

namespace rfqmix {

using namespace rfq;

constexpr int kLatPg = 32;
constexpr int kLatPad = 8;

template <int EK>
__global__ __launch_bounds__(256) void attn_latent_mfma_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride_t, int64_t q_stride_h,
    const bf16_t* __restrict__ pool, const int32_t* __restrict__ block_tables, int maxb,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ work_seq,
    const int32_t* __restrict__ work_qblk, bf16_t* __restrict__ out, int64_t out_stride,
    const float* __restrict__ sink, float scale, int H, int W, int nz) {
  constexpr int R = EK * 32, RS = R + kLatPad, VT = R / 16;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  bf16_t* c_lds = lds;                                 // [32][RS]
  // XCD-aware 1-D grid: consecutive workgroups go to the 8 XCDs in turn (each has its own L2),
  // so the nz workgroups of one work item -- they stream the same pages -- get ids 8 apart.
  const int n = blockIdx.x, k8 = n >> 3;
  const int wi = (k8 / nz) * 8 + (n & 7);
  const int bz = k8 % nz;
  if (wi >= W) return;
  const int s = work_seq[wi];
  if (s < 0) return;
  const int ql = q_len[s], kl = kv_len[s];
  const int i0 = work_qblk[wi] * 32;
  if (i0 >= ql) return;
  const int nq = min(32, ql - i0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (bz * 64 >= nq * H) return;                       // no column of this workgroup is used
  const int g4 = lane >> 4, c = lane & 15;
  const int tile = bz * 4 + wave;
  const bool active = tile * 16 < nq * H;              // wave-uniform
  const int col = tile * 16 + c;
  const int tok = col / H, hh = col - tok * H;
  const bool cvalid = active && tok < nq;
  const int p0 = kl - ql + i0, plast = p0 + nq - 1;
  const int pi = p0 + (cvalid ? tok : 0);
  const int32_t* bt = block_tables + (int64_t)s * maxb;

  // the lane's query column as B operands (k = 8 g4 + j of every 32-slice)
  s16x8 qf[EK];
  {
    const bf16_t* qp = q + (int64_t)(q_start[s] + i0 + (cvalid ? tok : 0)) * q_stride_t +
                       (int64_t)(cvalid ? hh : 0) * q_stride_h + 8 * g4;
#pragma unroll
    for (int k = 0; k < EK; ++k)
      qf[k] = cvalid ? *reinterpret_cast<const s16x8*>(qp + 32 * k) : (s16x8){0, 0, 0, 0, 0, 0, 0, 0};
  }
  f32x4 o[VT];
#pragma unroll
  for (int m = 0; m < VT; ++m) o[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m_run = (sink != nullptr && cvalid) ? sink[hh] : -INFINITY;
  float l_run = (sink != nullptr && cvalid) ? 1.f : 0.f;
  const bf16_t* ka = c_lds + c * RS + 8 * g4;          // this lane's A-fragment rows

  // Page pipeline: the next page is loaded into registers while this one is multiplied out of
  // LDS (one memory round trip per page, hidden behind the MFMAs).  Rows past the last key are
  // zeroed: they may hold anything, and 0 * NaN would poison the weighted sum.
  constexpr int NK = (kLatPg * (R / 8) + 255) / 256;
  s16x8 creg[NK];
  auto fetch = [&](int pg) {
    const s16x8* cb = reinterpret_cast<const s16x8*>(pool + (int64_t)bt[pg] * kLatPg * R);
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int x = threadIdx.x + u * 256;
      if (x < kLatPg * (R / 8))
        creg[u] = pg * kLatPg + x / (R / 8) > plast ? (s16x8){0, 0, 0, 0, 0, 0, 0, 0} : cb[x];
    }
  };
  const int pg_last = plast / kLatPg;
  fetch(0);
  for (int pg = 0; pg <= pg_last; ++pg) {
    const int kt = pg * kLatPg;
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int x = threadIdx.x + u * 256;
      if (x < kLatPg * (R / 8)) {
        const int row = x / (R / 8), x8 = x - row * (R / 8);
        *reinterpret_cast<s16x8*>(c_lds + row * RS + 8 * x8) = creg[u];
      }
    }
    __syncthreads();                                   // tile visible
    if (pg < pg_last) fetch(pg + 1);
    if (active) {
      constexpr int KF = EK < 8 ? EK : 8;
      f32x4 sc[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int k0 = 0; k0 < EK; k0 += KF) {
        s16x8 kf[2][KF];
#pragma unroll
        for (int k = 0; k < KF; ++k) {
          kf[0][k] = *reinterpret_cast<const s16x8*>(ka + 32 * (k0 + k));
          kf[1][k] = *reinterpret_cast<const s16x8*>(ka + 16 * RS + 32 * (k0 + k));
        }
        __builtin_amdgcn_sched_barrier(0);             // keep the reads ahead of the MFMAs
#pragma unroll
        for (int k = 0; k < KF; ++k) {
          sc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[0][k]), as_bf16x8(qf[k0 + k]),
                                                          sc[0], 0, 0, 0);
          sc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[1][k]), as_bf16x8(qf[k0 + k]),
                                                          sc[1], 0, 0, 0);
        }
      }
      // lane holds S^T[key = kt + 16 mt + 4 g4 + i][column c]
      float mx = -INFINITY;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kt + 16 * mt + 4 * g4 + i;
          const float v = (cvalid && key <= pi) ? sc[mt][i] * scale : -INFINITY;
          sc[mt][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __expf(m_run - m_use);
      float psum = 0.f, p[8];
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        p[jj] = __expf(sc[jj >> 2][jj & 3] - m_use);
        psum += p[jj];
      }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l_run = l_run * alpha + psum;
      m_run = m_new;
      // P^T as B operand: element j <-> key (j < 4 ? 4 g4 + j : 16 + 4 g4 + j - 4)
      u32x4 hb, lb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        hb[i] = pack_bf16x2(p[2 * i], p[2 * i + 1]);
        lb[i] = pack_bf16x2(p[2 * i] - __uint_as_float(hb[i] << 16),
                            p[2 * i + 1] - __uint_as_float(hb[i] & 0xffff0000u));
      }
      const s16x8 pb_hi = __builtin_bit_cast(s16x8, hb), pb_lo = __builtin_bit_cast(s16x8, lb);
      const int q4 = c >> 2, p4 = c & 3;
      const int r0 = 4 * g4 + q4, r1 = 16 + 4 * g4 + q4;
      // the accumulators are rescaled only on pages that moved some column's running maximum
      // (wave-uniform test; a factor of exactly 1 changes nothing)
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0ull) {
#pragma unroll
        for (int m = 0; m < VT; ++m) o[m] *= alpha;
      }
#pragma unroll
      for (int m = 0; m < VT; ++m) {
        const s16x4 a0 = ds_read_tr16(c_lds + r0 * RS + 16 * m + 4 * p4);
        const s16x4 a1 = ds_read_tr16(c_lds + r1 * RS + 16 * m + 4 * p4);
        const s16x8 a = (s16x8){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
        o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(pb_hi), o[m], 0, 0, 0);
        o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(pb_lo), o[m], 0, 0, 0);
      }
    }
    __syncthreads();                                   // before the next page overwrites the tile
  }
  if (!cvalid) return;
  // lane holds O^T[r = 16 m + 4 g4 + i][column c]
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  bf16_t* orow = out + (int64_t)(q_start[s] + i0 + tok) * out_stride + (int64_t)hh * R;
#pragma unroll
  for (int m = 0; m < VT; ++m) {
    uint2 w;
    w.x = pack_bf16x2(o[m][0] * inv, o[m][1] * inv);
    w.y = pack_bf16x2(o[m][2] * inv, o[m][3] * inv);
    *reinterpret_cast<uint2*>(orow + 16 * m + 4 * g4) = w;
  }
}

template <int EK>
static void launch_latent_one(const bf16_t* q, int64_t qst, int64_t qsh, const bf16_t* pool,
                              const int32_t* bt, int maxb, const int32_t* q_start,
                              const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                              const int32_t* work_qblk, int W, bf16_t* out, int64_t out_stride,
                              const float* sink, float scale, int H, hipStream_t s) {
  const int nz = (32 * H + 63) / 64;                   // workgroups of 64 columns per work item
  const size_t lds = (size_t)kLatPg * (EK * 32 + kLatPad) * sizeof(bf16_t);
  static bool attr = false;
  if (!attr) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_latent_mfma_kernel<EK>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  const dim3 grid(((W + 7) / 8) * 8 * nz);
  hipLaunchKernelGGL((attn_latent_mfma_kernel<EK>), grid, dim3(256), lds, s, q, qst, qsh, pool, bt,
                     maxb, q_start, q_len, kv_len, work_seq, work_qblk, out, out_stride, sink, scale,
                     H, W, nz);
}

// Sizes the tiles cover: 32-token pages, latent width 64, 128, 256 or 512.
bool latent_mfma_ok(int R, int BS) {
  return BS == kLatPg && (R == 64 || R == 128 || R == 256 || R == 512);
}

bool launch_attn_latent_mfma(const void* q, int64_t qst, int64_t qsh, const void* pool,
                             const int32_t* bt, int maxb, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                             const int32_t* work_qblk, int W, void* out, int64_t out_stride,
                             const float* sink, float scale, int H, int R, int BS, hipStream_t s) {
  if (!latent_mfma_ok(R, BS)) return false;
  if (W == 0) return true;
#define LAT_CASE(ek)                                                                            \
  if (R == 32 * ek) {                                                                           \
    launch_latent_one<ek>((const bf16_t*)q, qst, qsh, (const bf16_t*)pool, bt, maxb, q_start,   \
                          q_len, kv_len, work_seq, work_qblk, W, (bf16_t*)out, out_stride, sink, \
                          scale, H, s);                                                         \
    return true;                                                                                \
  }
  LAT_CASE(2) LAT_CASE(4) LAT_CASE(8) LAT_CASE(16)
#undef LAT_CASE
  return false;
}

}  // namespace rfqmix
