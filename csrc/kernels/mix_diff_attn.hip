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

}  // namespace rfqmix
