// Paged differential attention inside a sliding window.
//
// Every head holds two score maps: q [T, H, 2 dim] (fp32, already rotated) and the key pages
// [blocks, G, BS, 2 dim] carry map 1 in the first `dim` entries and map 2 in the rest; both
// maps weight the same value pages [blocks, G, BS, vdim].
//
//   s_m(i, j) = scale q_m(i) . k_m(j)          m = 1, 2;   i sees j <= i with i - j < window
//   a_m(i)    = sum_j softmax_j(s_m(i, .)) v(j)
//   o(i)      = a_1(i) - lam a_2(i)
//   out(i)    = o / sqrt(mean(o^2) + eps) * out_mult * sigmoid(gate(i, h))
//
// One workgroup per (work item, head); a work item is (sequence, block of QB queries), for
// prompt portions and for decode rows alike (a decode sequence is one item with few rows).
// Thread (ti, tj) of the 16 x 16 grid owns score rows ti, ti + 16 and columns tj + 16 k of a
// 64-key tile, for both maps; queries and keys pass through LDS in slices of EC dimensions.
// Scores, softmax, the weighted sums and the head norm are fp32 (FMA) for either cache type.
#include "mix_common.h"

namespace rfqmix {

namespace {
constexpr int DQB = 32;     // queries per work item
constexpr int DKT = 64;     // keys per tile
constexpr int DEC = 32;     // dimensions per LDS slice
constexpr float kNegInfD = -__builtin_huge_valf();
}  // namespace

template <typename T>
__global__ __launch_bounds__(256) void attn_diff_window_kernel(
    const float* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int maxb, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len,
    const int32_t* __restrict__ work_seq, const int32_t* __restrict__ work_qblk,
    const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out, int64_t out_stride,
    float scale, int window, float lam, float eps, float out_mult, int H, int G, int dim,
    int vdim, int BS) {
  const int s = work_seq[blockIdx.x];
  if (s < 0) return;
  const int hh = blockIdx.y;
  const int i0 = work_qblk[blockIdx.x] * DQB;
  const int ql = q_len[s];
  if (i0 >= ql) return;
  const int nq = min(DQB, ql - i0);
  const int p0 = kv_len[s] - ql + i0;                  // position of the block's first query
  const int plast = p0 + nq - 1;
  const int jlo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int g = hh / (H / G);
  const int kw = 2 * dim;
  const int tid = threadIdx.x;
  const int ti = tid >> 4, tj = tid & 15;

  extern __shared__ float lds[];
  float* Qs = lds;                                     // [DQB][DEC + 1]
  float* Ks = Qs + DQB * (DEC + 1);                    // [DKT][DEC + 1]
  float* Ps = Ks + DKT * (DEC + 1);                    // [2][DQB][DKT + 1]
  float* Os = Ps + 2 * DQB * (DKT + 1);                // [2][DQB][vdim]
  float* al = Os + 2 * DQB * vdim;                     // [2][DQB]
  float* ll = al + 2 * DQB;                            // [2][DQB]

  for (int x = tid; x < 2 * DQB * vdim; x += 256) Os[x] = 0.f;
  float m[2][2], l[2][2];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      m[mp][a] = kNegInfD;
      l[mp][a] = 0.f;
    }
  const float* qbase = q + ((int64_t)(q_start[s] + i0) * H + hh) * kw;

  for (int jb = jlo; jb <= plast; jb += DKT) {
    const int nk = min(DKT, plast + 1 - jb);
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      float sacc[2][4] = {};
      for (int e0 = 0; e0 < dim; e0 += DEC) {
        const int ne = min(DEC, dim - e0);
        __syncthreads();
        for (int x = tid; x < DQB * DEC; x += 256) {
          const int i = x / DEC, e = x - i * DEC;
          Qs[i * (DEC + 1) + e] =
              (i < nq && e < ne) ? qbase[(int64_t)i * H * kw + mp * dim + e0 + e] : 0.f;
        }
        for (int x = tid; x < DKT * DEC; x += 256) {
          const int jj = x / DEC, e = x - jj * DEC;
          float v = 0.f;
          if (jj < nk && e < ne) {
            const int j = jb + jj;
            v = ldf(k_cache + (((int64_t)bt[j / BS] * G + g) * BS + j % BS) * (int64_t)kw +
                    mp * dim + e0 + e);
          }
          Ks[jj * (DEC + 1) + e] = v;
        }
        __syncthreads();
        for (int e = 0; e < DEC; ++e) {
          const float q0 = Qs[ti * (DEC + 1) + e], q1 = Qs[(ti + 16) * (DEC + 1) + e];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float kv = Ks[(tj + 16 * k) * (DEC + 1) + e];
            sacc[0][k] += q0 * kv;
            sacc[1][k] += q1 * kv;
          }
        }
      }
      // scale, window mask, online softmax; a row's 64 columns live in the 16 lanes of its group
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int i = ti + 16 * a, pi = p0 + i;
        const int klo = window > 0 ? pi - window + 1 : 0;
        float mx = kNegInfD;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int j = jb + tj + 16 * k;
          const bool ok = i < nq && j <= pi && j >= klo;
          sacc[a][k] = ok ? sacc[a][k] * scale : kNegInfD;
          mx = fmaxf(mx, sacc[a][k]);
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float mn = fmaxf(m[mp][a], mx);
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float e = sacc[a][k] == kNegInfD ? 0.f : expf(sacc[a][k] - mn);
          Ps[(mp * DQB + i) * (DKT + 1) + tj + 16 * k] = e;
          sum += e;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        const float alpha = m[mp][a] == kNegInfD ? 0.f : expf(m[mp][a] - mn);
        l[mp][a] = l[mp][a] * alpha + sum;
        m[mp][a] = mn;
        if (tj == 0) al[mp * DQB + i] = alpha;
      }
    }
    __syncthreads();
    // both maps weight the same values: one pass over the tile's value rows
    for (int x = tid; x < nq * vdim; x += 256) {
      const int i = x / vdim, dv = x - i * vdim;
      float a0 = Os[x] * al[i], a1 = Os[DQB * vdim + x] * al[DQB + i];
      const float* p0r = Ps + i * (DKT + 1);
      const float* p1r = Ps + (DQB + i) * (DKT + 1);
      for (int jj = 0; jj < nk; ++jj) {
        const int j = jb + jj;
        const float v =
            ldf(v_cache + (((int64_t)bt[j / BS] * G + g) * BS + j % BS) * (int64_t)vdim + dv);
        a0 += p0r[jj] * v;
        a1 += p1r[jj] * v;
      }
      Os[x] = a0;
      Os[DQB * vdim + x] = a1;
    }
  }
  if (tj == 0) {
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      ll[mp * DQB + ti] = l[mp][0];
      ll[mp * DQB + ti + 16] = l[mp][1];
    }
  }
  __syncthreads();
  // o = a1 - lam a2 into the first accumulator
  for (int x = tid; x < nq * vdim; x += 256) {
    const int i = x / vdim;
    const float l0 = ll[i], l1 = ll[DQB + i];
    Os[x] = (l0 > 0.f ? Os[x] / l0 : 0.f) - lam * (l1 > 0.f ? Os[DQB * vdim + x] / l1 : 0.f);
  }
  __syncthreads();
  // head norm: eight lanes per row
  {
    const int i = tid >> 3, sub = tid & 7;
    float ss = 0.f;
    if (i < nq)
      for (int dv = sub; dv < vdim; dv += 8) {
        const float v = Os[i * vdim + dv];
        ss += v * v;
      }
#pragma unroll
    for (int o = 4; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (sub == 0 && i < nq) {
      const float gl = ldf(gate + (int64_t)(q_start[s] + i0 + i) * gate_stride + hh);
      al[i] = out_mult / sqrtf(ss / (float)vdim + eps) / (1.0f + expf(-gl));
    }
  }
  __syncthreads();
  for (int x = tid; x < nq * vdim; x += 256) {
    const int i = x / vdim, dv = x - i * vdim;
    stf(out + (int64_t)(q_start[s] + i0 + i) * out_stride + (int64_t)hh * vdim + dv,
        Os[x] * al[i]);
  }
}

// ------------------------------------------------------------------ decode rows
// One workgroup per (sequence, key/value head) and row of the short run: the rep = H / G heads
// of the group, two maps each, are R = 2 rep score rows over ONE pass through the group's
// key and value pages (a decode step streams every page once, not once per head).  A wave
// takes a score row at a time, a lane a key of the tile; the weighted sums of a tile are
// spread over all threads by (row, value channel).
// LDS (floats): qs[rep][kw] | Ks[KT][kw + 4 or 1] | Vs[KT][vdim] | Ps[R][KT] | acc[R][vdim] |
//               mrow[R] | lrow[R] | arow[R]
template <typename T>
__global__ __launch_bounds__(256) void attn_diff_decode_kernel(
    const float* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int maxb, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ kv_len,
    const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out, int64_t out_stride,
    float scale, int window, float lam, float eps, float out_mult, int H, int G, int dim,
    int vdim, int BS, int KT) {
  const int s = blockIdx.x, g = blockIdx.y;
  const int ql = q_len[s];
  const int32_t* bt = block_tables + (int64_t)s * maxb;
  const int rep = H / G, R = 2 * rep, kw = 2 * dim;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6, nw = blockDim.x >> 6;
  const int nthr = blockDim.x;

  // every region starts 16-byte aligned; with dim a multiple of 4 key rows are read in
  // 16-byte pieces (row stride kw + 4), else one float at a time (row stride kw + 1)
  const bool vec = (dim & 3) == 0;
  const int krs = kw + (vec ? 4 : 1);
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;
  float* Ks = qs + ((rep * kw + 3) & ~3);
  float* Vs = Ks + ((KT * krs + 3) & ~3);
  float* Ps = Vs + ((KT * vdim + 3) & ~3);
  float* acc = Ps + R * KT;
  float* mrow = acc + R * vdim;
  float* lrow = mrow + R;
  float* arow = lrow + R;

  // bf16 pages whose rows are whole 16-byte pieces: `width` values of key row jb + jj from
  // `cache` to dst[jj * dstride ...] as floats
  const bool vec8 = sizeof(T) == 2 && (kw & 7) == 0 && (vdim & 7) == 0 && (BS & (BS - 1)) == 0;
  const int bs_shift = 31 - __builtin_clz(BS);
  auto stage8 = [&](const T* cache, int width, int dstride, float* dst, int jb, int nk) {
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
          r[u] = *reinterpret_cast<const uint4*>(cache + rowi * width + c * 8);
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
  // the rows of a short run one after the other, gridDim.z of them at a time (a decode
  // step has one row per sequence: a grid over all possible rows would be mostly empty)
  for (int r = blockIdx.z; r < ql; r += gridDim.z) {
  const int t = q_start[s] + r;
  const int p = kv_len[s] - ql + r;                    // position of this row
  const int jlo = window > 0 ? max(0, p - window + 1) : 0;
  __syncthreads();                                     // the last row's reads are done
  for (int x = tid; x < rep * kw; x += nthr) qs[x] = q[((int64_t)t * H + g * rep) * kw + x];
  for (int x = tid; x < R * vdim; x += nthr) acc[x] = 0.f;
  for (int x = tid; x < R; x += nthr) {
    mrow[x] = kNegInfD;
    lrow[x] = 0.f;
  }

  for (int jb = jlo; jb <= p; jb += KT) {
    const int nk = min(KT, p + 1 - jb);
    __syncthreads();                                   // the last tile's sums are done
    bool staged = false;
    if constexpr (sizeof(T) == 2) {
      if (vec8) {
        // 16-byte pieces (8 values), four in flight per thread before the first is stored
        stage8(k_cache, kw, krs, Ks, jb, nk);
        stage8(v_cache, vdim, vdim, Vs, jb, nk);
        staged = true;
      }
    }
    if (!staged) {
      for (int jj = wid; jj < nk; jj += nw) {          // a wave per key row: one address per row
        const int j = jb + jj;
        const int64_t at = ((int64_t)bt[j / BS] * G + g) * BS + j % BS;
        const T* kr = k_cache + at * kw;
        const T* vr = v_cache + at * vdim;
        for (int e = lane; e < kw; e += 64) Ks[jj * krs + e] = ldf(kr + e);
        for (int e = lane; e < vdim; e += 64) Vs[jj * vdim + e] = ldf(vr + e);
      }
    }
    // the sums below walk the tile four keys at a time: rows past its end count as zeros
    for (int x = nk * vdim + tid; x < ((nk + 3) & ~3) * vdim; x += nthr) Vs[x] = 0.f;
    __syncthreads();
    for (int row = wid; row < R; row += nw) {
      const float* qv = qs + (row >> 1) * kw + (row & 1) * dim;
      float mx = kNegInfD;
      for (int jj = lane; jj < KT; jj += 64) {
        float a = kNegInfD;
        if (jj < nk) {
          const float* kv = Ks + jj * krs + (row & 1) * dim;
          float d0 = 0.f;
          if (vec) {
            for (int e = 0; e < dim; e += 4) {
              const float4 q4 = *reinterpret_cast<const float4*>(qv + e);
              const float4 k4 = *reinterpret_cast<const float4*>(kv + e);
              d0 += q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
            }
          } else {
            for (int e = 0; e < dim; ++e) d0 += qv[e] * kv[e];
          }
          a = d0 * scale;
        }
        Ps[row * KT + jj] = a;
        mx = fmaxf(mx, a);
      }
      mx = wave_max(mx);
      const float mo = mrow[row];
      const float mn = fmaxf(mo, mx);
      float sum = 0.f;
      for (int jj = lane; jj < KT; jj += 64) {
        const float v = Ps[row * KT + jj];
        const float e = v == kNegInfD ? 0.f : expf(v - mn);
        Ps[row * KT + jj] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float alpha = mo == kNegInfD ? 0.f : expf(mo - mn);
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
  }
  __syncthreads();
  for (int hr = wid; hr < rep; hr += nw) {
    const float l0 = lrow[2 * hr], l1 = lrow[2 * hr + 1];
    const float i0 = l0 > 0.f ? 1.0f / l0 : 0.f, i1 = l1 > 0.f ? lam / l1 : 0.f;
    float ss = 0.f;
    for (int dv = lane; dv < vdim; dv += 64) {
      const float o = acc[(2 * hr) * vdim + dv] * i0 - acc[(2 * hr + 1) * vdim + dv] * i1;
      ss += o * o;
    }
    ss = wave_sum(ss);
    const int hh = g * rep + hr;
    const float gl = ldf(gate + (int64_t)t * gate_stride + hh);
    const float mul = out_mult / sqrtf(ss / (float)vdim + eps) / (1.0f + expf(-gl));
    for (int dv = lane; dv < vdim; dv += 64) {
      const float o = acc[(2 * hr) * vdim + dv] * i0 - acc[(2 * hr + 1) * vdim + dv] * i1;
      stf(out + (int64_t)t * out_stride + (int64_t)hh * vdim + dv, o * mul);
    }
  }
  }
}

// ------------------------------------------------------------------ launcher
size_t attn_diff_lds(int vdim) {
  return ((size_t)DQB * (DEC + 1) + (size_t)DKT * (DEC + 1) + 2 * (size_t)DQB * (DKT + 1) +
          2 * (size_t)DQB * vdim + 4 * DQB) * sizeof(float);
}

bool launch_attn_diff_window(bool f32, const float* q, const void* k_cache, const void* v_cache,
                             const int32_t* bt, int maxb, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* kv_len, const int32_t* work_seq,
                             const int32_t* work_qblk, int W, const void* gate,
                             int64_t gate_stride, void* out, int64_t out_stride, float scale,
                             int window, float lam, float eps, float out_mult, int H, int G,
                             int dim, int vdim, int BS, hipStream_t s) {
  const size_t lds = attn_diff_lds(vdim);
  if (lds > (size_t)160 * 1024) return false;
  if (W == 0) return true;
  static bool attr = false;
  if (!attr) {          // dynamic LDS above 64 KB has to be allowed per kernel, once
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_diff_window_kernel<float>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_diff_window_kernel<bf16_t>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  if (f32)
    hipLaunchKernelGGL(attn_diff_window_kernel<float>, dim3(W, H), dim3(256), lds, s, q,
                       (const float*)k_cache, (const float*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, (const float*)gate, gate_stride, (float*)out,
                       out_stride, scale, window, lam, eps, out_mult, H, G, dim, vdim, BS);
  else
    hipLaunchKernelGGL(attn_diff_window_kernel<bf16_t>, dim3(W, H), dim3(256), lds, s, q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, work_seq, work_qblk, (const bf16_t*)gate, gate_stride, (bf16_t*)out,
                       out_stride, scale, window, lam, eps, out_mult, H, G, dim, vdim, BS);
  return true;
}

static size_t attn_diff_decode_floats(int rep, int dim, int vdim, int KT) {
  const int R = 2 * rep, kw = 2 * dim;
  return (size_t)rep * kw + 4 + (size_t)KT * (kw + 4) + 4 + (size_t)KT * vdim + 4 +
         (size_t)R * KT + (size_t)R * vdim + 3 * (size_t)R;
}

// Decode rows: one launch over (sequences, G, up to four rows at a time).  Returns the key tile used (0: the
// sizes do not fit the LDS; the caller then runs the work-item kernel).
int launch_attn_diff_decode(bool f32, const float* q, const void* k_cache, const void* v_cache,
                            const int32_t* bt, int maxb, const int32_t* q_start,
                            const int32_t* q_len, const int32_t* kv_len, int NA, int max_rows,
                            const void* gate, int64_t gate_stride, void* out, int64_t out_stride,
                            float scale, int window, float lam, float eps, float out_mult, int H,
                            int G, int dim, int vdim, int BS, hipStream_t s) {
  const int rep = H / G;
  // the largest key tile whose LDS fits two workgroups per CU, else one (160 KB per CU)
  int KT = 64;
  while (KT >= 16 && attn_diff_decode_floats(rep, dim, vdim, KT) * 4 > 80 * 1024) KT >>= 1;
  if (KT < 16) {
    KT = 64;
    while (KT >= 16 && attn_diff_decode_floats(rep, dim, vdim, KT) * 4 > 160 * 1024) KT >>= 1;
  }
  if (KT < 16) return 0;
  if (NA == 0) return KT;
  const size_t lds = attn_diff_decode_floats(rep, dim, vdim, KT) * 4;
  static bool attr = false;
  if (!attr) {
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_diff_decode_kernel<float>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_diff_decode_kernel<bf16_t>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  const dim3 grid(NA, G, max_rows < 4 ? max_rows : 4);
  if (f32)
    hipLaunchKernelGGL(attn_diff_decode_kernel<float>, grid, dim3(256), lds, s, q,
                       (const float*)k_cache, (const float*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, (const float*)gate, gate_stride, (float*)out, out_stride, scale,
                       window, lam, eps, out_mult, H, G, dim, vdim, BS, KT);
  else
    hipLaunchKernelGGL(attn_diff_decode_kernel<bf16_t>, grid, dim3(256), lds, s, q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, bt, maxb, q_start, q_len,
                       kv_len, (const bf16_t*)gate, gate_stride, (bf16_t*)out, out_stride, scale,
                       window, lam, eps, out_mult, H, G, dim, vdim, BS, KT);
  return KT;
}

}  // namespace rfqmix
