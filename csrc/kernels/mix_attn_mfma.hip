// MFMA attention of the layer-list models for bf16 caches (the math is at the top of
// mix_attn.hip).
//
// Head mixing is linear in the queries: with q~[h, c] = sum_{g in group c} (scale talk[h, g]) q_g
// the mixed score of head h is ONE product of q~[h, :] (E = G * dim wide) with the
// concatenation of all G key heads, and every head of a token reads the same keys.  A work
// item is (sequence, block of 32 query tokens, key/value head c); its columns are the
// (token, head) pairs of the heads that use value head c, 16 per wave:
//
//   prologue       q~ of the lane's column from the normed queries and the scaled mixing
//                  matrix, straight into B-operand registers (no mixed-query tensor in memory)
//   per 32-key page, shared by the workgroup's waves through LDS:
//     S^T[key, col]  = K_cat[key, :] . Q~[col, :]       v_mfma_f32_16x16x32_bf16, A = keys
//     bias, block mask, online softmax per column (fp32; the sink is the initial state)
//     O^T[dv, col]  += V_c^T[dv, key] . P^T[key, col]    A = V^T by transposed LDS reads,
//                                                        P split into bf16 hi + lo parts so
//                                                        the weights keep fp32's precision
//
// K and V rows are padded by 16 B in LDS so that the rows of a fragment read fall into
// different banks.  Two workgroups fit a compute unit (LDS and registers): one loads while the other
// multiplies.  The same kernel serves the decode section (one token x rep heads per tile).
#include "common.h"

namespace rfqmix {

using namespace rfq;

constexpr int kPg = 32;
constexpr int kKPad = 8;           // bf16 elements of padding per K / V row in LDS: row strides
                                   // of 16 B modulo 128 B, so the 8 lanes of a 16-byte read
                                   // phase (rows c .. c + 7) fall into different banks

// GRP (decode section): the four waves of a workgroup take four key/value heads (one column
// tile each) instead of four column tiles of one head, so the staged key page serves four
// times the heads; every wave stages its own head's V tile.
template <int EK, int VT, bool GRP>
__global__ __launch_bounds__(256) void attn_mixq_mfma_kernel(
    const float* __restrict__ qn, const float* __restrict__ ts, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int maxb,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ work_seq,
    const int32_t* __restrict__ work_qblk, bf16_t* __restrict__ out, int64_t out_stride,
    const float* __restrict__ slopes, const float* __restrict__ sink, int chunk, int H, int G,
    int dim, int W, int nz) {
  constexpr int VD = VT * 16, E = EK * 32, RS = E + kKPad, VRS = VD + kKPad;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  bf16_t* k_lds = lds;                       // [32][RS]
  bf16_t* v_lds = lds + kPg * RS;            // [32][VRS], one per wave with GRP
  // Work mapping.  GRP: grid (work item, group of four value heads, column tile).  Otherwise a
  // 1-D grid that is XCD-aware: consecutive workgroups go to the 8 XCDs in turn, and each XCD
  // has its own L2, so the G * nz workgroups of one work item (they all stream the same key
  // pages) get ids 8 apart -- same XCD, launched back to back -- and read each page from HBM /
  // MALL once and from that L2 otherwise.
  int wi, by, bz;
  if (GRP) {
    wi = blockIdx.x; by = blockIdx.y; bz = blockIdx.z;
  } else {
    const int n = blockIdx.x, per = G * nz, k = n >> 3;
    wi = (k / per) * 8 + (n & 7);
    const int yz = k % per;
    by = yz / nz; bz = yz - by * nz;
    if (wi >= W) return;
  }
  const int s = work_seq[wi];
  if (s < 0) return;
  const int ql = q_len[s], kl = kv_len[s];
  const int i0 = work_qblk[wi] * 32;
  if (i0 >= ql) return;
  const int nq = min(32, ql - i0);
  const int rep = H / G;
  const int nwaves = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if ((GRP ? bz : bz * nwaves) * 16 >= nq * rep) return;   // no column is used
  const int cg_raw = GRP ? by * 4 + wave : by;
  const int cg = cg_raw < G ? cg_raw : 0;
  const int g4 = lane >> 4, c = lane & 15;
  const int tile = GRP ? bz : bz * nwaves + wave;
  const bool active = cg_raw < G && tile * 16 < nq * rep;      // wave-uniform
  if (GRP) v_lds += wave * kPg * VRS;
  const int col = tile * 16 + c;
  const int tok = col / rep, hh = cg * rep + col % rep;
  const bool cvalid = active && tok < nq;
  const int p0 = kl - ql + i0, plast = p0 + nq - 1;
  const int pi = p0 + (cvalid ? tok : 0);
  const int klo = chunk > 0 ? (pi / chunk) * chunk : 0;      // first key of the query's block
  const int jlo = chunk > 0 ? (p0 / chunk) * chunk : 0;
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const float slope = slopes[hh];

  // mixed queries of this lane's column as B operands (k = 8 g4 + j of every 32-slice).  The
  // loop over the heads of a group has a run-time length, so it is the middle loop: each of
  // its rounds issues the loads of KB slices at once instead of one load per round trip.
  s16x8 qf[EK];
  {
    constexpr int KB = EK < 8 ? EK : 8;
    const float* qt = qn + (int64_t)(q_start[s] + i0 + (cvalid ? tok : 0)) * H * dim;
    const float* tr = ts + (int64_t)hh * H;
#pragma unroll
    for (int kg = 0; kg < EK; kg += KB) {
      float f[KB][8];
      int hq[KB], xo[KB];
#pragma unroll
      for (int k = 0; k < KB; ++k) {
        const int e0 = 32 * (kg + k) + 8 * g4, ck = e0 / dim;
        hq[k] = ck * rep;
        xo[k] = e0 - ck * dim;
#pragma unroll
        for (int j = 0; j < 8; ++j) f[k][j] = 0.f;
      }
      if (cvalid)
        for (int r = 0; r < rep; ++r) {
          float w[KB];
          float4 a[KB], b[KB];
#pragma unroll
          for (int k = 0; k < KB; ++k) {
            w[k] = tr[hq[k] + r];
            const float4* q4p = reinterpret_cast<const float4*>(qt + (int64_t)(hq[k] + r) * dim + xo[k]);
            a[k] = q4p[0];
            b[k] = q4p[1];
          }
#pragma unroll
          for (int k = 0; k < KB; ++k) {
            f[k][0] += w[k] * a[k].x; f[k][1] += w[k] * a[k].y;
            f[k][2] += w[k] * a[k].z; f[k][3] += w[k] * a[k].w;
            f[k][4] += w[k] * b[k].x; f[k][5] += w[k] * b[k].y;
            f[k][6] += w[k] * b[k].z; f[k][7] += w[k] * b[k].w;
          }
        }
#pragma unroll
      for (int k = 0; k < KB; ++k) qf[kg + k] = pack8(f[k]);
    }
  }
  f32x4 o[VT];
#pragma unroll
  for (int m = 0; m < VT; ++m) o[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m_run = (sink != nullptr && cvalid) ? sink[hh] : -INFINITY;
  float l_run = (sink != nullptr && cvalid) ? 1.f : 0.f;
  const bf16_t* ka = k_lds + c * RS + 8 * g4;          // this lane's A-fragment rows

  // Page pipeline: the next page's K / V pieces are loaded into registers while this page is
  // multiplied out of LDS (one memory round trip per page, hidden behind the MFMAs).
  constexpr int NK = (kPg * (E / 8) + 255) / 256;
  constexpr int VTHR = GRP ? 64 : 256, NV = (kPg * (VD / 8) + VTHR - 1) / VTHR;
  const int vtid = GRP ? lane : threadIdx.x;
  s16x8 kreg[NK], vreg[NV];
  int kdst[NK];                                        // LDS element offset of every K piece
  {
    const int d8 = dim >> 3;
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int x = threadIdx.x + u * 256;
      const int rowi = x / d8, x8 = x - rowi * d8, ck = rowi >> 5, key = rowi & 31;
      kdst[u] = x < kPg * (E / 8) ? key * RS + ck * dim + 8 * x8 : -1;
    }
  }
  auto fetch = [&](int pg) {
    const int64_t page = bt[pg];
    const s16x8* kb = reinterpret_cast<const s16x8*>(k_cache + page * G * kPg * (int64_t)dim);
    const s16x8* vb = reinterpret_cast<const s16x8*>(v_cache + ((page * G + cg) * kPg) * (int64_t)VD);
#pragma unroll
    for (int u = 0; u < NK; ++u)
      if (kdst[u] >= 0) kreg[u] = kb[threadIdx.x + u * 256];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int x = vtid + u * VTHR;
      // rows past the last written key are zeroed (they may hold anything, and 0 * NaN
      // would poison the sum)
      if (x < kPg * (VD / 8))
        vreg[u] = pg * kPg + x / (VD / 8) > plast ? (s16x8){0, 0, 0, 0, 0, 0, 0, 0} : vb[x];
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int u = 0; u < NK; ++u)
      if (kdst[u] >= 0) *reinterpret_cast<s16x8*>(k_lds + kdst[u]) = kreg[u];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int x = vtid + u * VTHR;
      if (x < kPg * (VD / 8))
        *reinterpret_cast<s16x8*>(v_lds + (x / (VD / 8)) * VRS + 8 * (x % (VD / 8))) = vreg[u];
    }
  };
  // GRP (few workgroups, one busy wave each) and the widest keys: the next page is loaded
  // into registers while this one is multiplied.  Otherwise a page is copied when it is needed
  // (fewer registers, more workgroups per compute unit that overlap each other); measured:
  // prefill of a 2048-wide, H 16 / G 4 layer 0.96 M tokens/s this way against 0.79-0.83 M
  // pipelined, of a 4096-wide, H 32 / G 8 layer 0.22 M against 0.26-0.27 M.
  constexpr bool PIPE = GRP || EK >= 32;
  const int pg_last = plast / kPg;
  if (PIPE) fetch(jlo / kPg);
  for (int pg = jlo / kPg; pg <= pg_last; ++pg) {
    const int kt = pg * kPg;
    if (PIPE) {
      stash();
    } else {
      // straight copy of the page's K heads (side by side) and of the V tile into LDS
      const int64_t page = bt[pg];
      const s16x8* kb = reinterpret_cast<const s16x8*>(k_cache + page * G * kPg * (int64_t)dim);
      const int d8 = dim >> 3;
      for (int x = threadIdx.x; x < kPg * (E / 8); x += 256) {
        const int rowi = x / d8, x8 = x - rowi * d8, ck = rowi >> 5, key = rowi & 31;
        *reinterpret_cast<s16x8*>(k_lds + key * RS + ck * dim + 8 * x8) = kb[x];
      }
      const s16x8* vb = reinterpret_cast<const s16x8*>(v_cache + ((page * G + cg) * kPg) * (int64_t)VD);
      for (int x = threadIdx.x; x < kPg * (VD / 8); x += 256) {
        const int row = x / (VD / 8);
        // rows past the last written key are zeroed (0 * NaN would poison the sum)
        const s16x8 v = kt + row > plast ? (s16x8){0, 0, 0, 0, 0, 0, 0, 0} : vb[x];
        *reinterpret_cast<s16x8*>(v_lds + row * VRS + 8 * (x % (VD / 8))) = v;
      }
    }
    __syncthreads();                                   // tiles visible
    if (PIPE && pg < pg_last) fetch(pg + 1);
    if (active) {
      // K fragments are read from LDS in batches of KF slices (both key halves) before the
      // MFMAs that use them, so the LDS latency is paid once per batch and not per MFMA
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
          const bool ok = cvalid && key <= pi && key >= klo;
          const float v = ok ? sc[mt][i] - slope * (float)(pi - key) : -INFINITY;
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
      // P^T as B operand: element j <-> key (j < 4 ? 4 g4 + j : 16 + 4 g4 + j - 4); hi = the
      // bf16 rounding of p (hardware conversion, two values per instruction), lo = bf16(p - hi)
      u32x4 hb, lb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        hb[i] = pack_bf16x2(p[2 * i], p[2 * i + 1]);
        lb[i] = pack_bf16x2(p[2 * i] - __uint_as_float(hb[i] << 16),
                            p[2 * i + 1] - __uint_as_float(hb[i] & 0xffff0000u));
      }
      const s16x8 pb_hi = __builtin_bit_cast(s16x8, hb), pb_lo = __builtin_bit_cast(s16x8, lb);
      const int q4 = c >> 2, p4 = c & 3;
#pragma unroll
      for (int m = 0; m < VT; ++m) {
        const int r0 = 4 * g4 + q4, r1 = 16 + 4 * g4 + q4;
        const s16x4 a0 = ds_read_tr16(v_lds + r0 * VRS + 16 * m + 4 * p4);
        const s16x4 a1 = ds_read_tr16(v_lds + r1 * VRS + 16 * m + 4 * p4);
        const s16x8 a = (s16x8){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
        o[m] *= alpha;
        o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(pb_hi), o[m], 0, 0, 0);
        o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(pb_lo), o[m], 0, 0, 0);
      }
    }
    __syncthreads();                                   // before the next page overwrites the tiles
  }
  if (!cvalid) return;
  // lane holds O^T[dv = 16 m + 4 g4 + i][column c]
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  bf16_t* orow = out + (int64_t)(q_start[s] + i0 + tok) * out_stride + (int64_t)hh * VD;
#pragma unroll
  for (int m = 0; m < VT; ++m) {
    uint2 w;
    w.x = pack_bf16x2(o[m][0] * inv, o[m][1] * inv);
    w.y = pack_bf16x2(o[m][2] * inv, o[m][3] * inv);
    *reinterpret_cast<uint2*>(orow + 16 * m + 4 * g4) = w;
  }
}

template <int EK, int VT, bool GRP>
static void launch_one(const float* qn, const float* ts, const bf16_t* k, const bf16_t* v, const int32_t* bt,
                       int maxb, const int32_t* q_start, const int32_t* q_len,
                       const int32_t* kv_len, const int32_t* work_seq, const int32_t* work_qblk,
                       int W, bf16_t* out, int64_t out_stride, const float* slopes,
                       const float* sink, int chunk, int H, int G, int dim, hipStream_t s) {
  const int rep = H / G;
  const int nwaves = 4;                  // waves without a column tile still load the pages
  const int z = GRP ? 2 * rep : (2 * rep + nwaves - 1) / nwaves;
  const int gy = GRP ? (G + 3) / 4 : G;
  const size_t lds = ((size_t)kPg * (EK * 32 + kKPad) +
                      (size_t)(GRP ? 4 : 1) * kPg * (VT * 16 + kKPad)) * sizeof(bf16_t);
  static bool attr = false;
  if (!attr) {          // dynamic LDS above 64 KB has to be allowed per kernel, once
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mixq_mfma_kernel<EK, VT, GRP>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  const dim3 grid = GRP ? dim3(W, gy, z) : dim3(((W + 7) / 8) * 8 * G * z);
  hipLaunchKernelGGL((attn_mixq_mfma_kernel<EK, VT, GRP>), grid, dim3(nwaves * 64), lds, s, qn,
                     ts, k, v, bt, maxb, q_start, q_len, kv_len, work_seq, work_qblk, out, out_stride,
                     slopes, sink, chunk, H, G, dim, W, z);
}

// Sizes the MFMA tiles cover: 32-token pages, dim a multiple of 32, E = G dim in
// {64, 128, 256, 512, 1024}, vdim in {32, 64, 128}, 16 a multiple of the heads per value head.
bool mixq_mfma_ok(int H, int G, int dim, int vdim, int BS) {
  const int rep = G > 0 ? H / G : 0, E = G * dim;
  return BS == kPg && rep >= 1 && H == rep * G && 16 % rep == 0 && dim % 32 == 0 &&
         (E == 64 || E == 128 || E == 256 || E == 512 || E == 1024) &&
         (vdim == 32 || vdim == 64 || vdim == 128) && G <= 65535;
}

bool launch_attn_mixq_prefill_mfma(const float* qn, const float* ts, const void* k_cache, const void* v_cache,
                                   const int32_t* bt, int maxb, const int32_t* q_start,
                                   const int32_t* q_len, const int32_t* kv_len,
                                   const int32_t* work_seq, const int32_t* work_qblk, int W,
                                   void* out, int64_t out_stride, const float* slopes,
                                   const float* sink, int chunk, int H, int G, int dim, int vdim,
                                   int BS, bool grouped, hipStream_t s) {
  if (!mixq_mfma_ok(H, G, dim, vdim, BS)) return false;
  if (W == 0) return true;
  const int EK = G * dim / 32, VT = vdim / 16;
#define MIXQ_CASE(ek, vt)                                                                       \
  if (EK == ek && VT == vt) {                                                                   \
    if (grouped)                                                                                \
      launch_one<ek, vt, true>(qn, ts, (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, \
                               q_start, q_len, kv_len, work_seq, work_qblk, W, (bf16_t*)out,   \
                               out_stride, slopes, sink, chunk, H, G, dim, s);                 \
    else                                                                                        \
      launch_one<ek, vt, false>(qn, ts, (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, \
                                q_start, q_len, kv_len, work_seq, work_qblk, W, (bf16_t*)out,  \
                                out_stride, slopes, sink, chunk, H, G, dim, s);                \
    return true;                                                                                \
  }
  MIXQ_CASE(2, 2) MIXQ_CASE(2, 4) MIXQ_CASE(2, 8)
  MIXQ_CASE(4, 2) MIXQ_CASE(4, 4) MIXQ_CASE(4, 8)
  MIXQ_CASE(8, 2) MIXQ_CASE(8, 4) MIXQ_CASE(8, 8)
  MIXQ_CASE(16, 2) MIXQ_CASE(16, 4) MIXQ_CASE(16, 8)
  MIXQ_CASE(32, 2) MIXQ_CASE(32, 4) MIXQ_CASE(32, 8)
#undef MIXQ_CASE
  return false;
}

}  // namespace rfqmix
