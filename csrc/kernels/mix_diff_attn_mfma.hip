// Differential attention inside a sliding window on MFMA tiles (bf16 pages, 32-token pages,
// map width a multiple of 32, value width a multiple of 16).  Semantics of mix_diff_attn.hip.
//
// One workgroup per (work item, head); a work item is (sequence, block of 32 queries).  Its
// four waves are (16 queries) x (score map): a wave keeps the online softmax of its map for
// its 16 query columns and the map's weighted values O_m^T [vdim x 16] in registers.  A key
// tile is one page: the head group's keys [32][2 dim] go to LDS as they lie in the page, its
// values likewise (read back transposed, ds_read_tr16_b64); the next page's pieces are
// loaded into registers while the current one is multiplied.
//
//   S^T[key, query] = K_m[key, :] . Q_m[query, :]    v_mfma_f32_16x16x32_bf16, A = key rows
//                     from LDS, B = the queries, held in registers as bf16 hi + lo parts (the
//                     rotated queries arrive in fp32 and are not rounded a second time)
//   scale, window mask, online softmax per query column in fp32
//   O^T[dv, query] += V^T[dv, keys] . P^T[keys, query]  A = two transposed reads of V, B = the
//                     weights straight from the score registers, as bf16 hi + lo parts (two
//                     MFMAs), so the weights keep fp32's precision.  The score tile leaves a
//                     lane with keys {4g .. 4g+3} of both 16-key halves; the A operand reads
//                     the same eight keys, so nothing is exchanged between lanes.
//
// Both maps' normalised sums meet in LDS: o = a1 - lam a2, head norm, gate, store.
#include "common.h"
#include "mix_common.h"

namespace rfqmix {

using rfq::as_bf16x8;
using rfq::f32x4;
using rfq::s16x4;
using rfq::s16x8;

namespace {
constexpr int MQB = 32;                 // queries per work item
constexpr int MBS = 32;                 // keys per tile = page size
constexpr float kNegInfM = -__builtin_huge_valf();

__device__ __forceinline__ void split_bf16(const float* f, s16x8& hi, s16x8& lo) {
  float r[8];
  hi = rfq::pack8(f);
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = f[i] - rfq::bf2f_s(hi[i]);
  lo = rfq::pack8(r);
}
}  // namespace

// DK = dim / 32 (score MFMAs per key half and part), DV = vdim / 16 (accumulator tiles).
template <int DK, int DV>
__global__ __launch_bounds__(256) void attn_diff_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int maxb,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ work_seq,
    const int32_t* __restrict__ work_qblk, const bf16_t* __restrict__ gate, int64_t gate_stride,
    bf16_t* __restrict__ out, int64_t out_stride, float scale, int window, float lam, float eps,
    float out_mult, int H, int G) {
  constexpr int dim = 32 * DK, vdim = 16 * DV, kw = 2 * dim;
  constexpr int KRS = kw + 8;            // shorts per key row in LDS (+ 16 bytes)
  constexpr int VRS = vdim + 8;          // shorts per value row
  const int s = work_seq[blockIdx.x];
  if (s < 0) return;
  const int hh = blockIdx.y;
  const int i0 = work_qblk[blockIdx.x] * MQB;
  const int ql = q_len[s];
  if (i0 >= ql) return;
  const int nq = min(MQB, ql - i0);
  const int p0 = kv_len[s] - ql + i0;
  const int plast = p0 + nq - 1;
  const int jlo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int g = hh / (H / G);
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int sub = wid & 1, mp = wid >> 1;
  const int col = lane & 15, grp = lane >> 4;
  const int row = sub * 16 + col;                        // this lane's query of the block
  const int pi = p0 + row;
  const int klo = window > 0 ? pi - window + 1 : 0;
  const bool qlive = row < nq;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  short* Ks = reinterpret_cast<short*>(smem);            // [32][KRS]
  short* Vs = Ks + MBS * KRS;                            // [32][VRS]
  // after the last tile the same memory holds both maps' sums, fp32 [2][32][vdim] + 64
  float* Os = reinterpret_cast<float*>(smem);
  float* al = Os + 2 * MQB * vdim;

  // the queries of this lane's column, as bf16 hi + lo parts
  s16x8 qhi[DK], qlo[DK];
  {
    const float* qp = q + ((int64_t)(q_start[s] + i0 + row) * H + hh) * kw + mp * dim + grp * 8;
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = qlive ? qp[ks * 32 + e] : 0.f;
      split_bf16(f, qhi[ks], qlo[ks]);
    }
  }
  f32x4 o[DV];
#pragma unroll
  for (int m = 0; m < DV; ++m) o[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float mrun = kNegInfM, lrun = 0.f;

  constexpr int NKV = (MBS * kw / 8 + 255) / 256, NVV = (MBS * vdim / 8 + 255) / 256;
  s16x8 kreg[NKV], vreg[NVV];
  auto fetch = [&](int pg) {
    const int64_t page = bt[pg];
    const s16x8* kp = reinterpret_cast<const s16x8*>(k_cache + ((page * G + g) * MBS) * (int64_t)kw);
    const s16x8* vp = reinterpret_cast<const s16x8*>(v_cache + ((page * G + g) * MBS) * (int64_t)vdim);
#pragma unroll
    for (int a = 0; a < NKV; ++a) {
      const int x = tid + a * 256;
      if (x < MBS * kw / 8) kreg[a] = kp[x];
    }
#pragma unroll
    for (int a = 0; a < NVV; ++a) {
      const int x = tid + a * 256;
      if (x < MBS * vdim / 8) vreg[a] = vp[x];
    }
  };
  const int pg_last = plast / MBS;
  fetch(jlo / MBS);
  for (int pg = jlo / MBS; pg <= pg_last; ++pg) {
    const int jb = pg * MBS;
    __syncthreads();                                     // the last tile's reads are done
#pragma unroll
    for (int a = 0; a < NKV; ++a) {
      const int x = tid + a * 256;
      if (x < MBS * kw / 8) {
        const int jj = x / (kw / 8), c = x - jj * (kw / 8);
        *reinterpret_cast<s16x8*>(Ks + jj * KRS + c * 8) = kreg[a];
      }
    }
#pragma unroll
    for (int a = 0; a < NVV; ++a) {
      const int x = tid + a * 256;
      if (x < MBS * vdim / 8) {
        const int jj = x / (vdim / 8), c = x - jj * (vdim / 8);
        s16x8 v = vreg[a];
        if (jb + jj > plast) v = (s16x8){0, 0, 0, 0, 0, 0, 0, 0};   // rows never written
        *reinterpret_cast<s16x8*>(Vs + jj * VRS + c * 8) = v;
      }
    }
    __syncthreads();
    if (pg < pg_last) fetch(pg + 1);                     // in flight during this tile's MFMAs
    // scores of the two 16-key halves
    f32x4 sc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      sc[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const short* kr = Ks + (kt * 16 + col) * KRS + mp * dim + grp * 8;
#pragma unroll
      for (int ks = 0; ks < DK; ++ks) {
        const s16x8 kf = *reinterpret_cast<const s16x8*>(kr + ks * 32);
        sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qhi[ks]), sc[kt], 0, 0, 0);
        sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qlo[ks]), sc[kt], 0, 0, 0);
      }
    }
    float mx = kNegInfM;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = jb + kt * 16 + grp * 4 + i;
        const bool ok = qlive && j <= pi && j >= klo;
        sc[kt][i] = ok ? sc[kt][i] * scale : kNegInfM;
        mx = fmaxf(mx, sc[kt][i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(mrun, mx);
    float pv[8], sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = sc[kt][i] == kNegInfM ? 0.f : __expf(sc[kt][i] - mn);
        pv[kt * 4 + i] = e;
        sum += e;
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float alpha = mrun == kNegInfM ? 0.f : __expf(mrun - mn);
    lrun = lrun * alpha + sum;
    mrun = mn;
    s16x8 phi, plo;
    split_bf16(pv, phi, plo);
    // the accumulators are rescaled only on pages that moved some column's running maximum
    // (wave-uniform test; a factor of exactly 1 changes nothing)
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0ull) {
#pragma unroll
      for (int m = 0; m < DV; ++m) o[m] *= alpha;
    }
    // transposed reads: a 16-lane group takes 4 key rows x 16 value columns, lane `col`
    // receives its column (keys 4 grp .. 4 grp + 3 of each 16-key half)
    const short* v0 = Vs + (4 * grp + (col >> 2)) * VRS + 4 * (col & 3);
    const short* v1 = v0 + 16 * VRS;
#pragma unroll
    for (int m = 0; m < DV; ++m) {
      const s16x4 a0 = rfq::ds_read_tr16(v0 + 16 * m);
      const s16x4 a1 = rfq::ds_read_tr16(v1 + 16 * m);
      const s16x8 a = (s16x8){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(phi), o[m], 0, 0, 0);
      o[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(plo), o[m], 0, 0, 0);
    }
  }
  __syncthreads();                                       // the tiles' LDS is free now
  {
    const float inv = lrun > 0.f ? 1.0f / lrun : 0.f;
    float* orow = Os + (mp * MQB + row) * vdim + grp * 4;
#pragma unroll
    for (int m = 0; m < DV; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) orow[m * 16 + i] = o[m][i] * inv;
  }
  __syncthreads();
  for (int x = tid; x < nq * vdim; x += 256) Os[x] = Os[x] - lam * Os[MQB * vdim + x];
  __syncthreads();
  {
    const int i = tid >> 3, sb = tid & 7;                // eight lanes per query row
    float ss = 0.f;
    if (i < nq)
      for (int dv = sb; dv < vdim; dv += 8) {
        const float v = Os[i * vdim + dv];
        ss += v * v;
      }
#pragma unroll
    for (int of = 4; of > 0; of >>= 1) ss += __shfl_xor(ss, of, 64);
    if (sb == 0 && i < nq) {
      const float gl = ldf(gate + (int64_t)(q_start[s] + i0 + i) * gate_stride + hh);
      al[i] = out_mult / sqrtf(ss / (float)vdim + eps) / (1.0f + expf(-gl));
    }
  }
  __syncthreads();
  for (int x = tid; x < nq * vdim; x += 256) {
    const int i = x / vdim, dv = x - i * vdim;
    stf(out + (int64_t)(q_start[s] + i0 + i) * out_stride + (int64_t)hh * vdim + dv, Os[x] * al[i]);
  }
}

// ------------------------------------------------------------------ launcher
bool diff_mfma_ok(int dim, int vdim, int BS) {
  return BS == MBS && (dim == 32 || dim == 64 || dim == 128) &&
         (vdim == 32 || vdim == 64 || vdim == 128);
}

template <int DK, int DV>
static void launch_diff_mfma_one(const float* q, const void* k_cache, const void* v_cache,
                                 const int32_t* bt, int maxb, const int32_t* q_start,
                                 const int32_t* q_len, const int32_t* kv_len,
                                 const int32_t* work_seq, const int32_t* work_qblk, int W,
                                 const void* gate, int64_t gate_stride, void* out,
                                 int64_t out_stride, float scale, int window, float lam, float eps,
                                 float out_mult, int H, int G, hipStream_t s) {
  constexpr int dim = 32 * DK, vdim = 16 * DV, kw = 2 * dim;
  const size_t tiles = (size_t)(MBS * (kw + 8) + MBS * (vdim + 8)) * 2;
  const size_t sums = (size_t)(2 * MQB * vdim + 64) * 4;
  const size_t lds = tiles > sums ? tiles : sums;
  static bool attr = false;
  if (!attr) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_diff_mfma_kernel<DK, DV>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  hipLaunchKernelGGL((attn_diff_mfma_kernel<DK, DV>), dim3(W, H), dim3(256), lds, s, q,
                     (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, q_start, q_len,
                     kv_len, work_seq, work_qblk, (const bf16_t*)gate, gate_stride, (bf16_t*)out,
                     out_stride, scale, window, lam, eps, out_mult, H, G);
}

bool launch_attn_diff_mfma(const float* q, const void* k_cache, const void* v_cache,
                           const int32_t* bt, int maxb, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                           const int32_t* work_qblk, int W, const void* gate, int64_t gate_stride,
                           void* out, int64_t out_stride, float scale, int window, float lam,
                           float eps, float out_mult, int H, int G, int dim, int vdim, int BS,
                           hipStream_t s) {
  if (!diff_mfma_ok(dim, vdim, BS)) return false;
  if (W == 0) return true;
#define DIFF_GO(DK, DV)                                                                          \
  launch_diff_mfma_one<DK, DV>(q, k_cache, v_cache, bt, maxb, q_start, q_len, kv_len, work_seq,  \
                               work_qblk, W, gate, gate_stride, out, out_stride, scale, window,  \
                               lam, eps, out_mult, H, G, s)
#define DIFF_DV(DK)                     \
  do {                                  \
    if (vdim == 32) DIFF_GO(DK, 2);     \
    else if (vdim == 64) DIFF_GO(DK, 4);\
    else DIFF_GO(DK, 8);                \
  } while (0)
  if (dim == 32) DIFF_DV(1);
  else if (dim == 64) DIFF_DV(2);
  else DIFF_DV(4);
#undef DIFF_DV
#undef DIFF_GO
  return true;
}

}  // namespace rfqmix
