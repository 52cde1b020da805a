// Projection norms with half-split rotation into the pages, and paged attention with a sliding
// window that keeps the first tokens, for softmax, sink-softmax and sigmoid weights.
//
//   qk_norm_rotary_append   rows q [H, qw] | k [G, kw] (| v [G, vdim]) of a fused projection:
//                           bias, RMS norm per head or over the whole projection, rotation of
//                           entries (off + i, off + i + n) by pos * f_i with a factor on cos and
//                           sin; q out in fp32, k and the values into their page rows
//   attn_keep_window        s(i, j) = scale q_h(i) . k_g(j);  i sees j <= i with
//                           i - j < window or j < keep_first (window 0: every j <= i)
//                             softmax:  w = exp(s) / (sum_j' exp(s(i, j')) [+ exp(bias_h)])
//                             sigmoid:  w = 1 / (1 + exp(-(s + bias_h))), not normalised
//                           out(i) = sum_j w v_g(j) [* sigmoid(gate(i, h))]
//                           The values are the first vdim entries of rows of stride vrs, so the
//                           key pages themselves can be the values (latent attention).
//   xielu_rows              z > 0: ap z^2 + z / 2;  z <= 0: an (exp(z) - 1 - z) + z / 2
//
// The attention kernels are the FMA forms (any sizes, fp32 or bf16 pages; scores, weights and
// sums in fp32): work items (sequence, block of QB queries) x head for prompt portions, one
// workgroup per (sequence, key/value head) over one pass through the pages for decode rows.
// MFMA tiles for bf16 pages are in mix_keep_attn_mfma.hip.
#include "mix_common.h"

namespace rfqmix {

namespace {
constexpr int KQB = 32;     // queries per work item
constexpr int KKT = 64;     // keys per tile
constexpr int KEC = 32;     // dimensions per LDS slice
constexpr float kNegInfK = -__builtin_huge_valf();
}  // namespace

// ------------------------------------------------------------------ norm, rotation, append
namespace {
// CW consecutive values as floats: CW = 8 moves 16 bytes of bf16 (32 of fp32) per access
template <int CW>
__device__ __forceinline__ void ld_chunk(const float* p, float* f) {
  if constexpr (CW == 8) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  } else {
    f[0] = *p;
  }
}
template <int CW>
__device__ __forceinline__ void ld_chunk(const bf16_t* p, float* f) {
  if constexpr (CW == 8) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(u[i] << 16);
      f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
    }
  } else {
    f[0] = ldf(p);
  }
}
template <int CW>
__device__ __forceinline__ void st_chunk(float* p, const float* f) {
  if constexpr (CW == 8) {
    *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
  } else {
    *p = f[0];
  }
}
template <int CW>
__device__ __forceinline__ void st_chunk(bf16_t* p, const float* f) {
  if constexpr (CW == 8) {
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bf16_t lo, hi;
      stf(&lo, f[2 * i]);
      stf(&hi, f[2 * i + 1]);
      u[i] = (uint32_t)lo | ((uint32_t)hi << 16);
    }
    *reinterpret_cast<uint4*>(p) = make_uint4(u[0], u[1], u[2], u[3]);
  } else {
    stf(p, f[0]);
  }
}
}  // namespace

// One workgroup per row; the row passes through LDS as floats.  CW = 8: every width, stride and
// pointer is a multiple of 8 values / 16 bytes, a thread moves chunks of 8 neighbouring values.
// LDS (floats): row[W] | fac[H + G] | cs[2 nrot] | scratch[16]
template <typename T, int CW>
__global__ __launch_bounds__(256) void qk_norm_rotary_append_kernel(
    const T* __restrict__ proj, int64_t stride, const float* __restrict__ bias,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, int norm_all,
    int k_norm_n, float eps, const int32_t* __restrict__ pos, const float* __restrict__ inv_freq,
    int nrot, float rot_mult, int q_rot_off, int k_rot_off, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int qw, int kw, int vdim,
    int v_mode, int BS, int64_t pool_slots, float* __restrict__ q_out) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int t = blockIdx.x, tid = threadIdx.x, nthr = blockDim.x;
  const int lane = tid & 63, wid = tid >> 6, nw = nthr >> 6;
  const int nq = H * qw, nk = G * kw;
  const int W = nq + nk + (v_mode == 0 ? G * vdim : 0);
  float* row = lds;
  float* fac = row + ((W + 3) & ~3);
  float* cs = fac + ((H + G + 3) & ~3);
  float* scratch = cs + 2 * nrot;

  // the row into LDS; with whole-projection norms the squares are summed on the way
  const T* src = proj + (int64_t)t * stride;
  float sq = 0.f, sk = 0.f;
  for (int c = tid * CW; c < W; c += nthr * CW) {
    float f[CW];
    ld_chunk<CW>(src + c, f);
    if (bias != nullptr) {
      float b[CW];
      ld_chunk<CW>(bias + c, b);
#pragma unroll
      for (int i = 0; i < CW; ++i) f[i] += b[i];
    }
    st_chunk<CW>(row + c, f);
    if (norm_all) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < CW; ++i) ss += f[i] * f[i];
      if (c < nq) sq += ss;
      else if (c < nq + nk) sk += ss;
    }
  }
  const float p = (float)pos[t];
  for (int i = tid; i < nrot; i += nthr) {
    float sn, c;
    sincosf(p * inv_freq[i], &sn, &c);
    cs[2 * i] = c * rot_mult;
    cs[2 * i + 1] = sn * rot_mult;
  }
  // norm factors: fac[0], fac[1] (whole projections) or one per head
  if (norm_all) {
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) {
      scratch[wid] = sq;
      scratch[8 + wid] = sk;
    }
    __syncthreads();
    if (tid == 0) {
      float a = 0.f, b = 0.f;
      for (int w = 0; w < nw; ++w) {
        a += scratch[w];
        b += scratch[8 + w];
      }
      fac[0] = q_norm_w != nullptr ? 1.0f / sqrtf(a / (float)nq + eps) : 1.f;
      fac[1] = k_norm_w != nullptr && nk > 0 ? 1.0f / sqrtf(b / (float)nk + eps) : 1.f;
    }
  } else {
    __syncthreads();
    // sixteen lanes per head: sixteen heads of the row are summed at a time
    const int sub = tid & 15, ngrp = nthr >> 4;
    for (int hd = tid >> 4; hd < H + G; hd += ngrp) {
      const bool isq = hd < H;
      const float* hv = isq ? row + hd * qw : row + nq + (hd - H) * kw;
      const int n = isq ? qw : k_norm_n;
      const bool normed = isq ? q_norm_w != nullptr : k_norm_w != nullptr;
      float ss = 0.f;
      if (normed)
        for (int e = sub; e < n; e += 16) ss += hv[e] * hv[e];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      if (sub == 0) fac[hd] = normed ? 1.0f / sqrtf(ss / (float)n + eps) : 1.f;
    }
  }
  __syncthreads();
  const int32_t slot = slots[t];
  const bool keep = G > 0 && slot >= 0 && slot < pool_slots;
  const int64_t page_row = keep ? ((int64_t)(slot / BS) * G) * BS + slot % BS : 0;   // + g * BS
  // the values: the keys as projected (mode 1) or the v columns (mode 0), neither normed nor rotated
  if (keep && v_mode != 2) {
    const float* vs = v_mode == 0 ? row + nq + nk : row + nq;
    for (int x = tid * CW; x < G * vdim; x += nthr * CW) {
      const int g = x / vdim, e = x - g * vdim;
      st_chunk<CW>(v_cache + (page_row + (int64_t)g * BS) * vdim + e, vs + x);
    }
  }
  // q and k: norm factor and weight, then the rotation (the partner entry is normed on the way).
  // CW = 8: the normed width, the rotation's offset and its half are multiples of 8, so a chunk
  // lies wholly inside or outside each of them and its partner chunk is one 32-byte LDS read.
  for (int c = tid * CW; c < nq + nk; c += nthr * CW) {
    const bool isq = c < nq;
    const int y = isq ? c : c - nq;
    const int width = isq ? qw : kw;
    const int hd = y / width, e = y - hd * width;
    const float* wv = isq ? q_norm_w : k_norm_w;
    const int nn = wv == nullptr ? 0 : (norm_all || isq ? width : k_norm_n);   // normed entries of a head
    const float fc = norm_all ? fac[isq ? 0 : 1] : fac[isq ? hd : H + hd];
    const float* wp = wv == nullptr ? nullptr : (norm_all ? wv + (y - e) : wv);  // the head's weights
    const int r0 = e - (isq ? q_rot_off : k_rot_off);
    float v[CW];
    if constexpr (CW == 8) {
      ld_chunk<8>(row + c, v);
      if (e < nn) {
        float w8[8];
        ld_chunk<8>(wp + e, w8);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] *= fc * w8[i];
      }
      if (r0 >= 0 && r0 < 2 * nrot) {
        const bool first = r0 < nrot;
        const int off = first ? nrot : -nrot, ii = first ? r0 : r0 - nrot;
        float u[8], c8[8], s8[8];
        ld_chunk<8>(row + c + off, u);
        if (e + off < nn) {
          float w8[8];
          ld_chunk<8>(wp + e + off, w8);
#pragma unroll
          for (int i = 0; i < 8; ++i) u[i] *= fc * w8[i];
        }
        ld_chunk<8>(cs + 2 * ii, c8);                 // (cos, sin) pairs ii .. ii + 3
        ld_chunk<8>(cs + 2 * ii + 8, s8);             // pairs ii + 4 .. ii + 7
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float cc = i < 4 ? c8[2 * i] : s8[2 * (i - 4)];
          const float sn = i < 4 ? c8[2 * i + 1] : s8[2 * (i - 4) + 1];
          v[i] = first ? v[i] * cc - u[i] * sn : v[i] * cc + u[i] * sn;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        const int ei = e + i, r = r0 + i;
        v[i] = row[c + i];
        if (ei < nn) v[i] *= fc * wp[ei];
        if (r >= 0 && r < 2 * nrot) {
          const int ii = r < nrot ? r : r - nrot;
          const int ej = r < nrot ? ei + nrot : ei - nrot;
          float u = row[c + i + (ej - ei)];
          if (ej < nn) u *= fc * wp[ej];
          const float cc = cs[2 * ii], sn = cs[2 * ii + 1];
          v[i] = r < nrot ? v[i] * cc - u * sn : v[i] * cc + u * sn;
        }
      }
    }
    if (isq)
      st_chunk<CW>(q_out + (int64_t)t * nq + c, v);
    else if (keep)
      st_chunk<CW>(k_cache + (page_row + (int64_t)hd * BS) * kw + e, v);
  }
}

// ------------------------------------------------------------------ prompt rows
// Work item (work_seq[w], work_qblk[w]) x head.  Thread (ti, tj) of the 16 x 16 grid owns score
// rows ti, ti + 16 and columns tj + 16 k of a 64-key tile; queries and keys pass through LDS in
// slices of KEC dimensions.  Key tiles cover the kept first tokens [0, kf) and then the
// window's range; nothing between them is read.
// LDS (floats): Qs[KQB][KEC+1] | Ks[KKT][KEC+1] | Ps[KQB][KKT+1] | Os[KQB][vdim] | al[KQB] | ll[KQB]
template <typename T>
__global__ __launch_bounds__(256) void attn_keep_window_kernel(
    const float* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    int64_t vrs, const int32_t* __restrict__ block_tables, int maxb,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const int32_t* __restrict__ work_seq,
    const int32_t* __restrict__ work_qblk, const float* __restrict__ head_bias,
    const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out, int64_t out_stride,
    float scale, int window, int keep_first, int sigmoid, int H, int G, int E, int vdim, int BS) {
  const int s = work_seq[blockIdx.x];
  if (s < 0) return;
  const int hh = blockIdx.y;
  const int i0 = work_qblk[blockIdx.x] * KQB;
  const int ql = q_len[s];
  if (i0 >= ql) return;
  const int nq = min(KQB, ql - i0);
  const int p0 = kv_len[s] - ql + i0;                  // position of the block's first query
  const int plast = p0 + nq - 1;
  const int jwin = window > 0 ? max(0, p0 - window + 1) : 0;
  const int kf = window > 0 ? min(keep_first, jwin) : 0;   // kept keys before the window
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int g = hh / (H / G);
  const int tid = threadIdx.x;
  const int ti = tid >> 4, tj = tid & 15;

  extern __shared__ float lds[];
  float* Qs = lds;
  float* Ks = Qs + KQB * (KEC + 1);
  float* Ps = Ks + KKT * (KEC + 1);
  float* Os = Ps + KQB * (KKT + 1);
  float* al = Os + KQB * vdim;
  float* ll = al + KQB;

  for (int x = tid; x < KQB * vdim; x += 256) Os[x] = 0.f;
  const float hb = head_bias != nullptr ? head_bias[hh] : 0.f;
  float m[2], l[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    m[a] = (!sigmoid && head_bias != nullptr) ? hb : kNegInfK;
    l[a] = (!sigmoid && head_bias != nullptr) ? 1.f : 0.f;
  }
  const float* qbase = q + ((int64_t)(q_start[s] + i0) * H + hh) * E;

  int jb = kf > 0 ? 0 : jwin;
  while (jb <= plast) {
    const bool head = jb < kf;
    const int nk = min(KKT, (head ? kf : plast + 1) - jb);
    float sacc[2][4] = {};
    for (int e0 = 0; e0 < E; e0 += KEC) {
      const int ne = min(KEC, E - e0);
      __syncthreads();
      for (int x = tid; x < KQB * KEC; x += 256) {
        const int i = x / KEC, e = x - i * KEC;
        Qs[i * (KEC + 1) + e] = (i < nq && e < ne) ? qbase[(int64_t)i * H * E + e0 + e] : 0.f;
      }
      for (int x = tid; x < KKT * KEC; x += 256) {
        const int jj = x / KEC, e = x - jj * KEC;
        float v = 0.f;
        if (jj < nk && e < ne) {
          const int j = jb + jj;
          v = ldf(k_cache + (((int64_t)bt[j / BS] * G + g) * BS + j % BS) * (int64_t)E + e0 + e);
        }
        Ks[jj * (KEC + 1) + e] = v;
      }
      __syncthreads();
      for (int e = 0; e < KEC; ++e) {
        const float q0 = Qs[ti * (KEC + 1) + e], q1 = Qs[(ti + 16) * (KEC + 1) + e];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float kv = Ks[(tj + 16 * k) * (KEC + 1) + e];
          sacc[0][k] += q0 * kv;
          sacc[1][k] += q1 * kv;
        }
      }
    }
    // scale, mask, weights; a row's 64 columns live in the 16 lanes of its group
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int i = ti + 16 * a, pi = p0 + i;
      float mx = kNegInfK;
      bool okk[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int jj = tj + 16 * k, j = jb + jj;
        okk[k] = i < nq && jj < nk && j <= pi && (window <= 0 || pi - j < window || j < keep_first);
        sacc[a][k] = okk[k] ? sacc[a][k] * scale : kNegInfK;
        mx = fmaxf(mx, sacc[a][k]);
      }
      float alpha = 1.f;
      if (sigmoid) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          Ps[i * (KKT + 1) + tj + 16 * k] = okk[k] ? 1.0f / (1.0f + expf(-(sacc[a][k] + hb))) : 0.f;
      } else {
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float mn = fmaxf(m[a], mx);
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float e = okk[k] ? expf(sacc[a][k] - mn) : 0.f;
          Ps[i * (KKT + 1) + tj + 16 * k] = e;
          sum += e;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        alpha = m[a] == kNegInfK ? 0.f : expf(m[a] - mn);
        l[a] = l[a] * alpha + sum;
        m[a] = mn;
      }
      if (tj == 0) al[i] = alpha;
    }
    __syncthreads();
    for (int x = tid; x < nq * vdim; x += 256) {
      const int i = x / vdim, dv = x - i * vdim;
      float acc = Os[x] * al[i];
      const float* pr = Ps + i * (KKT + 1);
      for (int jj = 0; jj < nk; ++jj) {
        const int j = jb + jj;
        acc += pr[jj] * ldf(v_cache + (((int64_t)bt[j / BS] * G + g) * BS + j % BS) * vrs + dv);
      }
      Os[x] = acc;
    }
    jb += nk;
    if (head && jb >= kf) jb = jwin;
  }
  if (tj == 0) {
    ll[ti] = l[0];
    ll[ti + 16] = l[1];
  }
  __syncthreads();
  for (int x = tid; x < nq * vdim; x += 256) {
    const int i = x / vdim, dv = x - i * vdim;
    const int64_t t = q_start[s] + i0 + i;
    float mul = sigmoid ? 1.f : (ll[i] > 0.f ? 1.0f / ll[i] : 0.f);
    if (gate != nullptr) mul /= 1.0f + expf(-ldf(gate + t * gate_stride + hh));
    stf(out + t * out_stride + (int64_t)hh * vdim + dv, Os[x] * mul);
  }
}

// ------------------------------------------------------------------ decode rows
// One workgroup per (sequence, key/value head) and row of the short run: the rep = H / G heads
// of the group are score rows over ONE pass through the group's key and value pages.  A wave
// takes a score row at a time, a lane a key of the tile; the weighted sums of a tile are spread
// over all threads by (rows, value channel).
// LDS (floats): qs[rep][E] | Ks[KT][E + 4 or 1] | Vs[KT][vdim] | Ps[rep][KT] | acc[rep][vdim] |
//               mrow[rep] | lrow[rep] | arow[rep]
template <typename T>
__global__ __launch_bounds__(256) void attn_keep_decode_kernel(
    const float* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    int64_t vrs, const int32_t* __restrict__ block_tables, int maxb,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ kv_len, const float* __restrict__ head_bias,
    const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out, int64_t out_stride,
    float scale, int window, int keep_first, int sigmoid, int H, int G, int E, int vdim, int BS,
    int KT) {
  const int s = blockIdx.x, g = blockIdx.y;
  const int ql = q_len[s];
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int R = H / G;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, nw = blockDim.x >> 6;
  const int nthr = blockDim.x;

  const bool vec = (E & 3) == 0;
  const int krs = E + (vec ? 4 : 1);
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;
  float* Ks = qs + ((R * E + 3) & ~3);
  float* Vs = Ks + ((KT * krs + 3) & ~3);
  float* Ps = Vs + ((KT * vdim + 3) & ~3);
  float* acc = Ps + R * KT;
  float* mrow = acc + R * vdim;
  float* lrow = mrow + R;
  float* arow = lrow + R;

  // bf16 pages whose rows are whole 16-byte pieces: `width` values of key row jb + jj from
  // rows of `rstride` values to dst[jj * dstride ...] as floats, four pieces in flight
  const bool vec8 = sizeof(T) == 2 && (E & 7) == 0 && (vdim & 7) == 0 && (vrs & 7) == 0 &&
                    (BS & (BS - 1)) == 0;
  const int bs_shift = 31 - __builtin_clz(BS);
  auto stage8 = [&](const T* cache, int64_t rstride, int width, int dstride, float* dst, int jb,
                    int nk) {
    const int w8 = width >> 3, total = nk * w8;
    for (int x0 = tid; x0 < total; x0 += 4 * nthr) {
      uint4 r[4];
      int at[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int x = x0 + u * nthr;
        at[u] = -1;
        if (x < total) {
          const int jj = x / w8, c = x - jj * w8, j = jb + jj;
          const int64_t rowi = ((int64_t)bt[j >> bs_shift] * G + g) * BS + (j & (BS - 1));
          r[u] = *reinterpret_cast<const uint4*>(cache + rowi * rstride + c * 8);
          at[u] = jj * dstride + c * 8;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (at[u] >= 0) {
          const uint32_t w[4] = {r[u].x, r[u].y, r[u].z, r[u].w};
          float f[8];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
          }
          *reinterpret_cast<float4*>(dst + at[u]) = make_float4(f[0], f[1], f[2], f[3]);
          *reinterpret_cast<float4*>(dst + at[u] + 4) = make_float4(f[4], f[5], f[6], f[7]);
        }
    }
  };
  for (int r = blockIdx.z; r < ql; r += gridDim.z) {
    const int t = q_start[s] + r;
    const int p = kv_len[s] - ql + r;                  // position of this row
    const int jwin = window > 0 ? max(0, p - window + 1) : 0;
    const int kf = window > 0 ? min(keep_first, jwin) : 0;
    __syncthreads();                                   // the last row's reads are done
    for (int x = tid; x < R * E; x += nthr) qs[x] = q[((int64_t)t * H + g * R) * E + x];
    for (int x = tid; x < R * vdim; x += nthr) acc[x] = 0.f;
    for (int x = tid; x < R; x += nthr) {
      const bool sk = !sigmoid && head_bias != nullptr;
      mrow[x] = sk ? head_bias[g * R + x] : kNegInfK;
      lrow[x] = sk ? 1.f : 0.f;
    }

    int jb = kf > 0 ? 0 : jwin;
    while (jb <= p) {
      const bool head = jb < kf;
      const int nk = min(KT, (head ? kf : p + 1) - jb);
      __syncthreads();                                 // the last tile's sums are done
      bool staged = false;
      if constexpr (sizeof(T) == 2) {
        if (vec8) {
          stage8(k_cache, E, E, krs, Ks, jb, nk);
          stage8(v_cache, vrs, vdim, vdim, Vs, jb, nk);
          staged = true;
        }
      }
      if (!staged) {
        for (int jj = wid; jj < nk; jj += nw) {        // a wave per key row: one address per row
          const int j = jb + jj;
          const int64_t at = ((int64_t)bt[j / BS] * G + g) * BS + j % BS;
          const T* kr = k_cache + at * E;
          const T* vr = v_cache + at * vrs;
          for (int e = lane; e < E; e += 64) Ks[jj * krs + e] = ldf(kr + e);
          for (int e = lane; e < vdim; e += 64) Vs[jj * vdim + e] = ldf(vr + e);
        }
      }
      // the sums below walk the tile four keys at a time: rows past its end count as zeros
      for (int x = nk * vdim + tid; x < ((nk + 3) & ~3) * vdim; x += nthr) Vs[x] = 0.f;
      __syncthreads();
      for (int row = wid; row < R; row += nw) {
        const float* qv = qs + row * E;
        const float hb = head_bias != nullptr ? head_bias[g * R + row] : 0.f;
        float mx = kNegInfK;
        for (int jj = lane; jj < KT; jj += 64) {
          float a = kNegInfK;
          if (jj < nk) {
            const float* kv = Ks + jj * krs;
            float d0 = 0.f;
            if (vec) {
              for (int e = 0; e < E; e += 4) {
                const float4 q4 = *reinterpret_cast<const float4*>(qv + e);
                const float4 k4 = *reinterpret_cast<const float4*>(kv + e);
                d0 += q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
              }
            } else {
              for (int e = 0; e < E; ++e) d0 += qv[e] * kv[e];
            }
            a = d0 * scale;
          }
          Ps[row * KT + jj] = a;
          mx = fmaxf(mx, a);
        }
        if (sigmoid) {
          for (int jj = lane; jj < KT; jj += 64) {
            const float v = Ps[row * KT + jj];
            Ps[row * KT + jj] = v == kNegInfK ? 0.f : 1.0f / (1.0f + expf(-(v + hb)));
          }
          if (lane == 0) arow[row] = 1.f;
          continue;
        }
        mx = wave_max(mx);
        const float mo = mrow[row];
        const float mn = fmaxf(mo, mx);
        float sum = 0.f;
        for (int jj = lane; jj < KT; jj += 64) {
          const float v = Ps[row * KT + jj];
          const float e = v == kNegInfK ? 0.f : expf(v - mn);
          Ps[row * KT + jj] = e;
          sum += e;
        }
        sum = wave_sum(sum);
        if (lane == 0) {
          const float alpha = mo == kNegInfK ? 0.f : expf(mo - mn);
          arow[row] = alpha;
          lrow[row] = lrow[row] * alpha + sum;
          mrow[row] = mn;
        }
      }
      __syncthreads();
      // a thread takes a value channel and up to four score rows: a value is read once for all
      // of them, the weights of four keys in one 16-byte read
      const int RG = (R + 3) >> 2;
      for (int x = tid; x < vdim * RG; x += nthr) {
        const int rg = x / vdim, dv = x - rg * vdim;
        const int r0 = rg * 4, nr = min(4, R - r0);
        float a[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = i < nr ? acc[(r0 + i) * vdim + dv] * arow[r0 + i] : 0.f;
        for (int jj = 0; jj < nk; jj += 4) {
          const float v0 = Vs[jj * vdim + dv], v1 = Vs[(jj + 1) * vdim + dv];
          const float v2 = Vs[(jj + 2) * vdim + dv], v3 = Vs[(jj + 3) * vdim + dv];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (i < nr) {
              const float4 p4 = *reinterpret_cast<const float4*>(Ps + (r0 + i) * KT + jj);
              a[i] += p4.x * v0 + p4.y * v1 + p4.z * v2 + p4.w * v3;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (i < nr) acc[(r0 + i) * vdim + dv] = a[i];
      }
      jb += nk;
      if (head && jb >= kf) jb = jwin;
    }
    __syncthreads();
    for (int hr = wid; hr < R; hr += nw) {
      const int hh = g * R + hr;
      float mul = sigmoid ? 1.f : (lrow[hr] > 0.f ? 1.0f / lrow[hr] : 0.f);
      if (gate != nullptr) mul /= 1.0f + expf(-ldf(gate + (int64_t)t * gate_stride + hh));
      for (int dv = lane; dv < vdim; dv += 64)
        stf(out + (int64_t)t * out_stride + (int64_t)hh * vdim + dv, acc[hr * vdim + dv] * mul);
    }
  }
}

// ------------------------------------------------------------------ xIELU
template <typename T, int CW>
__global__ __launch_bounds__(256) void xielu_rows_kernel(const T* __restrict__ x, int64_t xs,
                                                         T* __restrict__ out, int64_t os, int F,
                                                         float ap, float an) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * CW;
  if (c >= F) return;
  float z[CW], y[CW];
  ld_chunk<CW>(x + (int64_t)t * xs + c, z);
#pragma unroll
  for (int i = 0; i < CW; ++i)
    y[i] = z[i] > 0.f ? ap * z[i] * z[i] + 0.5f * z[i] : an * (expm1f(z[i]) - z[i]) + 0.5f * z[i];
  st_chunk<CW>(out + (int64_t)t * os + c, y);
}

// ------------------------------------------------------------------ launchers
namespace {
constexpr int kLdsMax = 160 * 1024;
template <typename K>
void allow_lds(K kernel) {
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax);
}
}  // namespace

bool launch_qk_norm_rotary_append(bool f32, const void* proj, int64_t stride, const float* bias,
                                  const float* q_norm_w, const float* k_norm_w, bool norm_all,
                                  int k_norm_n, float eps, const int32_t* pos,
                                  const float* inv_freq, int nrot, float rot_mult, int q_rot_off,
                                  int k_rot_off, const int32_t* slots, void* k_cache, void* v_cache,
                                  int T, int H, int G, int qw, int kw, int vdim, int v_mode, int BS,
                                  int64_t pool_slots, float* q_out, hipStream_t s) {
  const size_t W = (size_t)H * qw + (size_t)G * kw + (v_mode == 0 ? (size_t)G * vdim : 0);
  const size_t lds = (W + 4 + H + G + 4 + 2 * (size_t)nrot + 16) * sizeof(float);
  if (lds > (size_t)kLdsMax) return false;
  if (T == 0) return true;
  static bool attr = false;
  if (!attr) {
    allow_lds(&qk_norm_rotary_append_kernel<float, 1>);
    allow_lds(&qk_norm_rotary_append_kernel<bf16_t, 1>);
    allow_lds(&qk_norm_rotary_append_kernel<float, 8>);
    allow_lds(&qk_norm_rotary_append_kernel<bf16_t, 8>);
    attr = true;
  }
  auto al16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = qw % 8 == 0 && (G == 0 || kw % 8 == 0) && (v_mode == 2 || vdim % 8 == 0) &&
                   stride % 8 == 0 && k_norm_n % 8 == 0 && nrot % 8 == 0 && q_rot_off % 8 == 0 &&
                   k_rot_off % 8 == 0 && al16(proj) && al16(bias) && al16(q_norm_w) &&
                   al16(k_norm_w) && al16(k_cache) && al16(v_cache) && al16(q_out);
#define QKN_GO(TT, CW)                                                                          \
  hipLaunchKernelGGL((qk_norm_rotary_append_kernel<TT, CW>), dim3(T), dim3(256), lds, s,       \
                     (const TT*)proj, stride, bias, q_norm_w, k_norm_w, (int)norm_all, k_norm_n, \
                     eps, pos, inv_freq, nrot, rot_mult, q_rot_off, k_rot_off, slots,           \
                     (TT*)k_cache, (TT*)v_cache, H, G, qw, kw, vdim, v_mode, BS, pool_slots, q_out)
  if (f32) {
    if (vec) QKN_GO(float, 8);
    else QKN_GO(float, 1);
  } else {
    if (vec) QKN_GO(bf16_t, 8);
    else QKN_GO(bf16_t, 1);
  }
#undef QKN_GO
  return true;
}

bool launch_attn_keep_window(bool f32, const float* q, const void* k_cache, const void* v_cache,
                             int64_t vrs, const int32_t* bt, int maxb, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                             const int32_t* work_qblk, int W, const float* head_bias,
                             const void* gate, int64_t gate_stride, void* out, int64_t out_stride,
                             float scale, int window, int keep_first, bool sigmoid, int H, int G,
                             int E, int vdim, int BS, hipStream_t s) {
  const size_t lds = ((size_t)KQB * (KEC + 1) + (size_t)KKT * (KEC + 1) + (size_t)KQB * (KKT + 1) +
                      (size_t)KQB * vdim + 2 * KQB) * sizeof(float);
  if (lds > (size_t)kLdsMax) return false;
  if (W == 0) return true;
  static bool attr = false;
  if (!attr) {
    allow_lds(&attn_keep_window_kernel<float>);
    allow_lds(&attn_keep_window_kernel<bf16_t>);
    attr = true;
  }
  if (f32)
    hipLaunchKernelGGL(attn_keep_window_kernel<float>, dim3(W, H), dim3(256), lds, s, q,
                       (const float*)k_cache, (const float*)v_cache, vrs, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, head_bias, (const float*)gate, gate_stride,
                       (float*)out, out_stride, scale, window, keep_first, (int)sigmoid, H, G, E,
                       vdim, BS);
  else
    hipLaunchKernelGGL(attn_keep_window_kernel<bf16_t>, dim3(W, H), dim3(256), lds, s, q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, vrs, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, head_bias, (const bf16_t*)gate, gate_stride,
                       (bf16_t*)out, out_stride, scale, window, keep_first, (int)sigmoid, H, G, E,
                       vdim, BS);
  return true;
}

static size_t attn_keep_decode_floats(int R, int E, int vdim, int KT) {
  return (size_t)R * E + 4 + (size_t)KT * (E + 4) + 4 + (size_t)KT * vdim + 4 + (size_t)R * KT +
         (size_t)R * vdim + 3 * (size_t)R;
}

// Decode rows: one launch over (sequences, G, up to four rows at a time).  Returns the key tile
// used (0: the sizes do not fit the LDS; the caller then runs the work-item kernel).
int launch_attn_keep_decode(bool f32, const float* q, const void* k_cache, const void* v_cache,
                            int64_t vrs, const int32_t* bt, int maxb, const int32_t* q_start,
                            const int32_t* q_len, const int32_t* kv_len, int NA, int max_rows,
                            const float* head_bias, const void* gate, int64_t gate_stride, void* out,
                            int64_t out_stride, float scale, int window, int keep_first,
                            bool sigmoid, int H, int G, int E, int vdim, int BS, hipStream_t s) {
  const int R = H / G;
  int KT = 64;
  while (KT >= 16 && attn_keep_decode_floats(R, E, vdim, KT) * 4 > 80 * 1024) KT >>= 1;
  if (KT < 16) {
    KT = 64;
    while (KT >= 16 && attn_keep_decode_floats(R, E, vdim, KT) * 4 > (size_t)kLdsMax) KT >>= 1;
  }
  if (KT < 16) return 0;
  if (NA == 0) return KT;
  const size_t lds = attn_keep_decode_floats(R, E, vdim, KT) * 4;
  static bool attr = false;
  if (!attr) {
    allow_lds(&attn_keep_decode_kernel<float>);
    allow_lds(&attn_keep_decode_kernel<bf16_t>);
    attr = true;
  }
  const dim3 grid(NA, G, max_rows < 4 ? max_rows : 4);
  if (f32)
    hipLaunchKernelGGL(attn_keep_decode_kernel<float>, grid, dim3(256), lds, s, q,
                       (const float*)k_cache, (const float*)v_cache, vrs, bt, maxb, q_start, q_len,
                       kv_len, head_bias, (const float*)gate, gate_stride, (float*)out, out_stride,
                       scale, window, keep_first, (int)sigmoid, H, G, E, vdim, BS, KT);
  else
    hipLaunchKernelGGL(attn_keep_decode_kernel<bf16_t>, grid, dim3(256), lds, s, q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, vrs, bt, maxb, q_start, q_len,
                       kv_len, head_bias, (const bf16_t*)gate, gate_stride, (bf16_t*)out, out_stride,
                       scale, window, keep_first, (int)sigmoid, H, G, E, vdim, BS, KT);
  return KT;
}

void launch_xielu_rows(bool f32, const void* x, int64_t xs, void* out, int64_t os, int T, int F,
                       float ap, float an, hipStream_t s) {
  if (T == 0 || F == 0) return;
  const bool vec = F % 8 == 0 && xs % 8 == 0 && os % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int per = vec ? 2048 : 256;
  const dim3 grid(T, (F + per - 1) / per);
#define XI_GO(TT, CW)                                                                        \
  hipLaunchKernelGGL((xielu_rows_kernel<TT, CW>), grid, dim3(256), 0, s, (const TT*)x, xs,  \
                     (TT*)out, os, F, ap, an)
  if (f32) {
    if (vec) XI_GO(float, 8);
    else XI_GO(float, 1);
  } else {
    if (vec) XI_GO(bf16_t, 8);
    else XI_GO(bf16_t, 1);
  }
#undef XI_GO
}

}  // namespace rfqmix
