// attn_keep_window on MFMA tiles (bf16 pages of 32 tokens, key width a multiple of 32, value
// width a multiple of 16).  Semantics of mix_keep_attn.hip: sliding window with kept first
// tokens; softmax, softmax with a sink, or unnormalised sigmoid weights; optional output gate;
// the values may be the leading entries of the key rows themselves (latent attention).
//
// One workgroup per (work item, HPW heads of one key/value head); a work item is (sequence,
// block of 32 queries).  Its 2 HPW waves are (16 queries) x (head): a wave keeps the running
// maximum and sum of its 16 query columns and the weighted values O^T [vdim x 16] in
// registers.  A key tile is one page: the head group's key rows go to LDS as they lie in the
// page, its value rows likewise (read back transposed, ds_read_tr16_b64); with shared pages
// the key rows are staged once and read both ways.  The next page's pieces are loaded into
// registers while the current one is multiplied.  Pages between the kept first tokens and the
// window are never read.
//
// Decode rows (DEC): a workgroup takes one row of a sequence at a time and its 16 columns per
// wave are 16 HEADS of one key/value head, so the pages of a sequence are streamed once for 32
// heads (latent attention: all heads share the one key head) instead of once per head pair.
//
//   S^T[key, query] = K[key, :] . Q[query, :]   v_mfma_f32_16x16x32_bf16, A = key rows from LDS,
//                     B = the queries in registers as bf16 hi (+ lo for keys of up to 320
//                     entries: they arrive in fp32 and are not rounded a second time)
//   scale, mask, weights per query column in fp32
//   O^T[dv, query] += V^T[dv, keys] . P^T[keys, query]   A = two transposed reads of V, B = the
//                     weights straight from the score registers as bf16 hi + lo parts (two
//                     MFMAs), so the weights keep fp32's precision
#include "common.h"
#include "mix_common.h"

namespace rfqmix {

using rfq::as_bf16x8;
using rfq::f32x4;
using rfq::s16x4;
using rfq::s16x8;

namespace {
constexpr int WQB = 32;                 // queries per work item
constexpr int WBS = 32;                 // keys per tile = page size
constexpr float kNegInfW = -__builtin_huge_valf();

__device__ __forceinline__ void split_bf16w(const float* f, s16x8& hi, s16x8& lo) {
  float r[8];
  hi = rfq::pack8(f);
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = f[i] - rfq::bf2f_s(hi[i]);
  lo = rfq::pack8(r);
}
}  // namespace

// DK = E / 32, DV = vdim / 16, HPW heads per workgroup, SHARED: values = leading entries of the
// key rows, QLO: the queries' lo parts are multiplied too, DEC: decode rows (grid = sequences x
// (key/value head, block of 32 heads) x rows in flight; no work lists).
template <int DK, int DV, int HPW, bool SHARED, bool QLO, bool DEC>
__global__ __launch_bounds__(128 * HPW) void attn_keep_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, int64_t vrs, const int32_t* __restrict__ block_tables,
    int maxb, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ work_seq,
    const int32_t* __restrict__ work_qblk, const float* __restrict__ head_bias,
    const bf16_t* __restrict__ gate, int64_t gate_stride, bf16_t* __restrict__ out,
    int64_t out_stride, float scale, int window, int keep_first, int sigmoid, int H, int G) {
  constexpr int E = 32 * DK, vdim = 16 * DV, NT = 128 * HPW;
  constexpr int KRS = E + 8;                       // shorts per key row in LDS (+ 16 bytes)
  constexpr int VRS = SHARED ? KRS : vdim + 8;     // shorts per value row
  const int s = DEC ? (int)blockIdx.x : work_seq[blockIdx.x];
  if (s < 0) return;
  const int ql = q_len[s];
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int rep = H / G;
  // prompt rows: columns are 16 queries of head hh; decode rows: 16 heads of one row
  const int per_g = (rep + 32 * HPW - 1) / (32 * HPW);
  const int ho = DEC ? ((int)blockIdx.y % per_g) * 32 * HPW + wid * 16 + col : 0;
  const int g = DEC ? (int)blockIdx.y / per_g : ((int)blockIdx.y * HPW) / rep;
  const int hh = DEC ? g * rep + min(ho, rep - 1) : (int)blockIdx.y * HPW + (wid >> 1);
  const int i0 = DEC ? 0 : work_qblk[blockIdx.x] * WQB;
  if (!DEC && i0 >= ql) return;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  short* Ks = reinterpret_cast<short*>(smem);      // [32][KRS]
  short* Vs = SHARED ? Ks : Ks + WBS * KRS;        // [32][VRS]

  for (int r = DEC ? (int)blockIdx.z : 0; r < (DEC ? ql : 1); r += DEC ? (int)gridDim.z : 1) {
  const int nq = DEC ? 1 : min(WQB, ql - i0);
  const int p0 = kv_len[s] - ql + (DEC ? r : i0);
  const int plast = p0 + nq - 1;
  const int jwin = window > 0 ? max(0, p0 - window + 1) : 0;
  const int kf = window > 0 ? min(keep_first, jwin) : 0;     // kept keys before the window
  const int row = DEC ? r : (wid & 1) * 16 + col;  // this lane's query of the run / block
  const int pi = DEC ? p0 : p0 + row;
  const bool qlive = DEC ? ho < rep : row < nq;
  const int64_t t = q_start[s] + i0 + row;

  s16x8 qhi[DK], qlo[QLO ? DK : 1];
  {
    const float* qp = q + (t * H + hh) * E + grp * 8;
#pragma unroll
    for (int ks = 0; ks < DK; ++ks) {
      float f[8];
      if (qlive) {
        const float4 a = *reinterpret_cast<const float4*>(qp + ks * 32);
        const float4 b = *reinterpret_cast<const float4*>(qp + ks * 32 + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = 0.f;
      }
      if constexpr (QLO) {
        split_bf16w(f, qhi[ks], qlo[ks]);
      } else {
        qhi[ks] = rfq::pack8(f);
      }
    }
  }
  f32x4 o[DV];
#pragma unroll
  for (int m = 0; m < DV; ++m) o[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const float hb = head_bias != nullptr ? head_bias[hh] : 0.f;
  const bool sink = !sigmoid && head_bias != nullptr;
  float mrun = sink ? hb : kNegInfW, lrun = sink ? 1.f : 0.f;

  constexpr int NKV = (WBS * E / 8 + NT - 1) / NT;
  constexpr int NVV = SHARED ? 1 : (WBS * vdim / 8 + NT - 1) / NT;
  s16x8 kreg[NKV], vreg[NVV];
  auto fetch = [&](int pg) {
    const int64_t page = bt[pg];
    const s16x8* kp = reinterpret_cast<const s16x8*>(k_cache + ((page * G + g) * WBS) * (int64_t)E);
#pragma unroll
    for (int a = 0; a < NKV; ++a) {
      const int x = tid + a * NT;
      if (x < WBS * E / 8) kreg[a] = kp[x];
    }
    if constexpr (!SHARED) {
      const bf16_t* vb = v_cache + ((page * G + g) * WBS) * vrs;
#pragma unroll
      for (int a = 0; a < NVV; ++a) {
        const int x = tid + a * NT;
        if (x < WBS * vdim / 8) {
          const int jj = x / (vdim / 8), c = x - jj * (vdim / 8);
          vreg[a] = *reinterpret_cast<const s16x8*>(vb + jj * vrs + c * 8);
        }
      }
    }
  };
  // pages [0 .. pg_keep] hold the kept first tokens, pages [pg_win .. pg_last] the window
  const int pg_last = plast / WBS;
  const int pg_keep = kf > 0 ? (kf - 1) / WBS : -1;
  const int pg_win = jwin / WBS;
  auto next_page = [&](int pg) { return (pg == pg_keep && pg_win > pg) ? pg_win : pg + 1; };
  int pg = kf > 0 ? 0 : pg_win;
  fetch(pg);
  while (pg <= pg_last) {
    const int jb = pg * WBS;
    const int pg_next = next_page(pg);
    __syncthreads();                                     // the last tile's reads are done
#pragma unroll
    for (int a = 0; a < NKV; ++a) {
      const int x = tid + a * NT;
      if (x < WBS * E / 8) {
        const int jj = x / (E / 8), c = x - jj * (E / 8);
        s16x8 v = kreg[a];
        if (SHARED && jb + jj > plast) v = (s16x8){0, 0, 0, 0, 0, 0, 0, 0};   // rows never written
        *reinterpret_cast<s16x8*>(Ks + jj * KRS + c * 8) = v;
      }
    }
    if constexpr (!SHARED) {
#pragma unroll
      for (int a = 0; a < NVV; ++a) {
        const int x = tid + a * NT;
        if (x < WBS * vdim / 8) {
          const int jj = x / (vdim / 8), c = x - jj * (vdim / 8);
          s16x8 v = vreg[a];
          if (jb + jj > plast) v = (s16x8){0, 0, 0, 0, 0, 0, 0, 0};
          *reinterpret_cast<s16x8*>(Vs + jj * VRS + c * 8) = v;
        }
      }
    }
    __syncthreads();
    if (pg_next <= pg_last) fetch(pg_next);              // in flight during this tile's MFMAs
    // scores of the two 16-key halves
    f32x4 sc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      sc[kt] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const short* kr = Ks + (kt * 16 + col) * KRS + grp * 8;
#pragma unroll
      for (int ks = 0; ks < DK; ++ks) {
        const s16x8 kfr = *reinterpret_cast<const s16x8*>(kr + ks * 32);
        sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kfr), as_bf16x8(qhi[ks]), sc[kt], 0, 0, 0);
        if constexpr (QLO)
          sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kfr), as_bf16x8(qlo[ks]), sc[kt], 0, 0, 0);
      }
    }
    float pv[8];
    float alpha = 1.f;
    if (sigmoid) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = jb + kt * 16 + grp * 4 + i;
          const bool ok = qlive && j <= pi && (window <= 0 || pi - j < window || j < keep_first);
          pv[kt * 4 + i] = ok ? 1.0f / (1.0f + __expf(-(sc[kt][i] * scale + hb))) : 0.f;
        }
    } else {
      float mx = kNegInfW;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = jb + kt * 16 + grp * 4 + i;
          const bool ok = qlive && j <= pi && (window <= 0 || pi - j < window || j < keep_first);
          sc[kt][i] = ok ? sc[kt][i] * scale : kNegInfW;
          mx = fmaxf(mx, sc[kt][i]);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(mrun, mx);
      float sum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = sc[kt][i] == kNegInfW ? 0.f : __expf(sc[kt][i] - mn);
          pv[kt * 4 + i] = e;
          sum += e;
        }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      alpha = mrun == kNegInfW ? 0.f : __expf(mrun - mn);
      lrun = lrun * alpha + sum;
      mrun = mn;
    }
    s16x8 phi, plo;
    split_bf16w(pv, phi, plo);
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
    pg = pg_next;
  }
  // lane (col, grp) holds value channels 16 m + 4 grp .. + 3 of its column: 8-byte stores
  if (qlive) {
    float mul = sigmoid ? 1.f : (lrun > 0.f ? 1.0f / lrun : 0.f);
    if (gate != nullptr) mul /= 1.0f + __expf(-ldf(gate + t * gate_stride + hh));
    bf16_t* orow = out + t * out_stride + (int64_t)hh * vdim + grp * 4;
#pragma unroll
    for (int m = 0; m < DV; ++m) {
      bf16_t b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) stf(&b[i], o[m][i] * mul);
      *reinterpret_cast<uint2*>(orow + m * 16) =
          make_uint2((uint32_t)b[0] | ((uint32_t)b[1] << 16), (uint32_t)b[2] | ((uint32_t)b[3] << 16));
    }
  }
  }
}

// ------------------------------------------------------------------ launcher
namespace {
bool plain_sizes(int DK, int DV) { return DK >= 1 && DK <= 4 && (DV == 2 || DV == 4 || DV == 8); }
bool shared_sizes(int DK, int DV) {
  return (DK == 3 && DV == 4) || (DK == 5 && DV == 8) || (DK == 6 && DV == 8) ||
         (DK == 10 && DV == 16) || (DK == 18 && DV == 32);
}
}  // namespace

bool keep_mfma_ok(int E, int vdim, int BS, bool shared) {
  if (BS != WBS || E % 32 != 0 || vdim % 16 != 0) return false;
  return shared ? shared_sizes(E / 32, vdim / 16) : plain_sizes(E / 32, vdim / 16);
}

struct KeepArgs {
  const float* q;
  const void *k_cache, *v_cache;
  int64_t vrs;
  const int32_t *bt;
  int maxb;
  const int32_t *q_start, *q_len, *kv_len, *work_seq, *work_qblk;
  int W;
  const float* head_bias;
  const void* gate;
  int64_t gate_stride;
  void* out;
  int64_t out_stride;
  float scale;
  int window, keep_first;
  bool sigmoid;
  int H, G;
  int NA, short_rows;      // decode rows: sequences, and the most rows any of them has (0: work items)
  hipStream_t s;
};

template <int DK, int DV, int HPW, bool SHARED, bool DEC>
static void launch_keep_mfma_one(const KeepArgs& a) {
  constexpr bool QLO = DK <= 10;       // wider keys: the queries' registers go to the accumulators
  constexpr int E = 32 * DK, vdim = 16 * DV;
  const size_t lds = (size_t)(WBS * (E + 8) + (SHARED ? 0 : WBS * (vdim + 8))) * 2;
  static bool attr = false;
  if (!attr) {
    (void)hipFuncSetAttribute(
        reinterpret_cast<const void*>(&attn_keep_mfma_kernel<DK, DV, HPW, SHARED, QLO, DEC>),
        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  const int rep = a.H / a.G;
  const dim3 grid = DEC ? dim3(a.NA, a.G * ((rep + 32 * HPW - 1) / (32 * HPW)),
                               a.short_rows < 4 ? a.short_rows : 4)
                        : dim3(a.W, a.H / HPW);
  hipLaunchKernelGGL((attn_keep_mfma_kernel<DK, DV, HPW, SHARED, QLO, DEC>), grid,
                     dim3(128 * HPW), lds, a.s, a.q, (const bf16_t*)a.k_cache,
                     (const bf16_t*)a.v_cache, a.vrs, a.bt, a.maxb, a.q_start, a.q_len, a.kv_len,
                     a.work_seq, a.work_qblk, a.head_bias, (const bf16_t*)a.gate, a.gate_stride,
                     (bf16_t*)a.out, a.out_stride, a.scale, a.window, a.keep_first, (int)a.sigmoid,
                     a.H, a.G);
}

template <int DK, int DV, bool SHARED>
static void launch_keep_mfma_heads(const KeepArgs& a) {
  if (a.short_rows > 0) launch_keep_mfma_one<DK, DV, 1, SHARED, true>(a);
  else if ((a.H / a.G) % 2 == 0) launch_keep_mfma_one<DK, DV, 2, SHARED, false>(a);
  else launch_keep_mfma_one<DK, DV, 1, SHARED, false>(a);
}

bool launch_attn_keep_mfma(const float* q, const void* k_cache, const void* v_cache, int64_t vrs,
                           const int32_t* bt, int maxb, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                           const int32_t* work_qblk, int W, const float* head_bias,
                           const void* gate, int64_t gate_stride, void* out, int64_t out_stride,
                           float scale, int window, int keep_first, bool sigmoid, int H, int G,
                           int E, int vdim, int BS, bool shared, int NA, int short_rows,
                           hipStream_t s) {
  if (!keep_mfma_ok(E, vdim, BS, shared)) return false;
  if (short_rows > 0 ? NA == 0 : W == 0) return true;
  const KeepArgs a{q, k_cache, v_cache, vrs, bt, maxb, q_start, q_len, kv_len, work_seq, work_qblk,
                   W, head_bias, gate, gate_stride, out, out_stride, scale, window, keep_first,
                   sigmoid, H, G, NA, short_rows, s};
  const int DK = E / 32, DV = vdim / 16;
  if (shared) {
    if (DK == 3) launch_keep_mfma_heads<3, 4, true>(a);
    else if (DK == 5) launch_keep_mfma_heads<5, 8, true>(a);
    else if (DK == 6) launch_keep_mfma_heads<6, 8, true>(a);
    else if (DK == 10) launch_keep_mfma_heads<10, 16, true>(a);
    else launch_keep_mfma_heads<18, 32, true>(a);
    return true;
  }
#define KEEP_DV(DKK)                                                    \
  do {                                                                  \
    if (DV == 2) launch_keep_mfma_heads<DKK, 2, false>(a);              \
    else if (DV == 4) launch_keep_mfma_heads<DKK, 4, false>(a);         \
    else launch_keep_mfma_heads<DKK, 8, false>(a);                      \
  } while (0)
  if (DK == 1) KEEP_DV(1);
  else if (DK == 2) KEEP_DV(2);
  else if (DK == 3) KEEP_DV(3);
  else KEEP_DV(4);
#undef KEEP_DV
  return true;
}

}  // namespace rfqmix
