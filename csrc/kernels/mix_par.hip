// Row kernels of parallel-sublayer layers and their mixers' pre-processing:
//
//   residual_add_norm   x += mult (y1 + y2) + shift (fp32 stream), then h = rms(x) (w + offset) for
//                       the next layer: one kernel per layer boundary
//   rotary_append       interleaved-pair rotation of the leading dimensions of every score
//                       map of q and k; k and v into their pages, q out in fp32
//   conv_act_heads      causal convolution over time + silu of projection outputs, with the
//                       last taps - 1 inputs kept per sequence; leading heads made unit vectors
//   moe_route_topk      largest router logits (+ bias), softmax over the chosen ones
//   gelu_rows           exact gelu
//
// One workgroup per token row (the router: one thread per row).  Norms, angles, the stream,
// the convolution state and the router are fp32 whatever the activation type is.
#include "mix_common.h"

namespace rfqmix {

__device__ __forceinline__ float ld_any(const void* p, bool f32, int64_t i) {
  return f32 ? static_cast<const float*>(p)[i] : ldf(static_cast<const bf16_t*>(p) + i);
}

// x[t] += mult (y1[t] + y2[t]) + shift; out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * (w + offset).
// y1, y2, shift and (w, out) are each optional; y1 / y2 are fp32 or bf16 (flags).
template <typename TO>
__global__ __launch_bounds__(256) void residual_add_norm_kernel(
    float* __restrict__ x, const void* __restrict__ y1, int64_t y1_stride, bool y1_f32,
    const void* __restrict__ y2, int64_t y2_stride, bool y2_f32, const float* __restrict__ shift,
    const float* __restrict__ w, float eps, float offset, TO* __restrict__ out, int d, float mult) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float y = 0.f;
    if (y1 != nullptr) y += ld_any(y1, y1_f32, (int64_t)t * y1_stride + c);
    if (y2 != nullptr) y += ld_any(y2, y2_f32, (int64_t)t * y2_stride + c);
    float v = xr[c] + y * mult;
    if (shift != nullptr) v += shift[c];
    xr[c] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)d + eps);
  // every thread re-reads the entries it wrote itself
  for (int c = threadIdx.x; c < d; c += blockDim.x)
    stf(out + (int64_t)t * d + c, xr[c] * r * (w[c] + offset));
}

// Row t of qkv = q [H][maps][dim] | k [G][maps][dim] | v [G][vdim].  Entries (2i, 2i+1),
// i < nrot, of every map of q and k turn by the angle pos * inv_freq[i].
template <typename T>
__global__ __launch_bounds__(256) void rotary_append_kernel(
    const T* __restrict__ qkv, int64_t stride, const int32_t* __restrict__ pos,
    const float* __restrict__ inv_freq, int nrot, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int maps, int dim, int vdim,
    int BS, int64_t pool_slots, float* __restrict__ q_out) {
  extern __shared__ float cs[];                      // [nrot] of (cos, sin): one per pair index
  const int t = blockIdx.x;
  const T* row = qkv + (int64_t)t * stride;
  const float p = (float)pos[t];
  // the angle depends on the pair index only: every head and map reuses the row's sines
  for (int i = threadIdx.x; i < nrot; i += blockDim.x) {
    float sn, c;
    sincosf(p * inv_freq[i], &sn, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = sn;
  }
  __syncthreads();
  const int32_t slot = slots[t];
  const bool keep = slot >= 0 && slot < pool_slots;
  const int half = dim / 2 + (dim & 1);              // pairs per map (+ a lone last entry)
  const int nqp = H * maps * half, nkp = G * maps * half;
  const int kw = maps * dim;
  for (int x = threadIdx.x; x < nqp + nkp; x += blockDim.x) {
    const bool is_q = x < nqp;
    const int y = is_q ? x : x - nqp;
    const int hm = y / half, i = y - hm * half;      // (head, map) and pair index
    const int e = hm * dim + 2 * i;                  // offset inside q or k
    const T* src = row + (is_q ? 0 : H * kw) + e;
    const bool pair = 2 * i + 1 < dim;
    float u = ldf(src), v = pair ? ldf(src + 1) : 0.f;
    if (i < nrot && pair) {
      const float c = cs[2 * i], sn = cs[2 * i + 1];
      const float a = u * c - v * sn, b = v * c + u * sn;
      u = a;
      v = b;
    }
    if (is_q) {
      float* o = q_out + (int64_t)t * H * kw + e;
      o[0] = u;
      if (pair) o[1] = v;
    } else if (keep) {
      const int g = hm / maps, off = e - g * kw;
      T* o = k_cache + (((int64_t)(slot / BS) * G + g) * BS + slot % BS) * (int64_t)kw + off;
      stf(o, u);
      if (pair) stf(o + 1, v);
    }
  }
  if (keep) {
    const T* vs = row + (int64_t)(H + G) * kw;
    for (int x = threadIdx.x; x < G * vdim; x += blockDim.x) {
      const int g = x / vdim, e = x - g * vdim;
      v_cache[(((int64_t)(slot / BS) * G + g) * BS + slot % BS) * (int64_t)vdim + e] = vs[x];
    }
  }
}

// Eight entries (four pairs) per thread: dim, vdim and the row stride multiples of 8, 16-byte
// aligned rows and pages.
__device__ __forceinline__ void ld8any(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void ld8any(const bf16_t* p, float* f) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(u[i] << 16);
    f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void st8any(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
__device__ __forceinline__ void st8any(bf16_t* p, const float* f) {
  uint32_t u[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bf16_t lo, hi;
    stf(&lo, f[2 * i]);
    stf(&hi, f[2 * i + 1]);
    u[i] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
  *reinterpret_cast<uint4*>(p) = make_uint4(u[0], u[1], u[2], u[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void rotary_append_vec_kernel(
    const T* __restrict__ qkv, int64_t stride, const int32_t* __restrict__ pos,
    const float* __restrict__ inv_freq, int nrot, const int32_t* __restrict__ slots,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int maps, int dim, int vdim,
    int BS, int64_t pool_slots, float* __restrict__ q_out) {
  extern __shared__ float cs[];
  const int t = blockIdx.x;
  const T* row = qkv + (int64_t)t * stride;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; i < nrot; i += blockDim.x) {
    float sn, c;
    sincosf(p * inv_freq[i], &sn, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = sn;
  }
  __syncthreads();
  const int32_t slot = slots[t];
  const bool keep = slot >= 0 && slot < pool_slots;
  const int d8 = dim >> 3, kw = maps * dim;
  const int nq8 = H * maps * d8, nk8 = G * maps * d8, nv8 = (G * vdim) >> 3;
  const int64_t prow = keep ? ((int64_t)(slot / BS) * G) * BS + slot % BS : 0;   // + g * BS per head
  for (int x = threadIdx.x; x < nq8 + nk8 + nv8; x += blockDim.x) {
    float f[8];
    if (x >= nq8 + nk8) {                              // values: a plain copy into the page
      if (!keep) continue;
      const int y = (x - nq8 - nk8) * 8, g = y / vdim, e = y - g * vdim;
      ld8any(row + (int64_t)(H + G) * kw + y, f);
      st8any(v_cache + (prow + (int64_t)g * BS) * vdim + e, f);
      continue;
    }
    const bool is_q = x < nq8;
    const int y = is_q ? x : x - nq8;
    const int hm = y / d8, i0 = (y - hm * d8) * 4;     // (head, map), first pair index
    const int e = hm * dim + 2 * i0;
    ld8any(row + (is_q ? 0 : H * kw) + e, f);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i0 + u < nrot) {
        const float c = cs[2 * (i0 + u)], sn = cs[2 * (i0 + u) + 1];
        const float a = f[2 * u] * c - f[2 * u + 1] * sn, b = f[2 * u + 1] * c + f[2 * u] * sn;
        f[2 * u] = a;
        f[2 * u + 1] = b;
      }
    if (is_q) {
      st8any(q_out + (int64_t)t * H * kw + e, f);
    } else if (keep) {
      const int g = hm / maps, off = e - g * kw;
      st8any(k_cache + (prow + (int64_t)g * BS) * kw + off, f);
    }
  }
}

// y[t, c] = silu(sum_j w[c, j] x[t - (taps-1-j), c]); rows before the run come from the
// sequence's state half, rows before position 0 are zero; the run's last taps - 1 inputs go
// to the other half.  Then heads [0, n_unit) of `dim` channels become unit vectors.
// A workgroup takes `chunk` channels (a multiple of dim, so no head straddles two) of a row.
// LDS: chunk floats.
template <typename T>
__global__ __launch_bounds__(256) void conv_act_heads_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
    float* __restrict__ state, const int32_t* __restrict__ row_state,
    const int32_t* __restrict__ row_back, const int32_t* __restrict__ row_fwd,
    const int32_t* __restrict__ pos, float* __restrict__ out, int C, int taps, int slots,
    int n_unit, int dim, float unit_eps, int chunk) {
  extern __shared__ float ys[];
  const int t = blockIdx.x;
  const int c0 = blockIdx.y * chunk;
  const int nc = min(chunk, C - c0);
  const int code = row_state[t], i = row_back[t], f = row_fwd[t], p = pos[t];
  const int K = taps - 1;
  const float* rd = code >= 0 ? state + ((int64_t)((code & 1) * slots + (code >> 1)) * K) * C : nullptr;
  float* wr = code >= 0 ? state + ((int64_t)((1 - (code & 1)) * slots + (code >> 1)) * K) * C : nullptr;
  const T* xr = x + (int64_t)t * x_stride;
  const int n = i + f + 1;
  for (int cc = threadIdx.x; cc < nc; cc += blockDim.x) {
    const int c = c0 + cc;
    const float x0 = ldf(xr + c);
    const float* wc = w + (int64_t)c * taps;
    float acc = wc[taps - 1] * x0;
    for (int dl = 1; dl < taps; ++dl) {
      float src;
      if (dl <= i) src = ldf(xr - (int64_t)dl * x_stride + c);
      else if (p - dl >= 0 && rd != nullptr) src = rd[(int64_t)(K + i - dl) * C + c];
      else continue;
      acc += wc[taps - 1 - dl] * src;
    }
    ys[cc] = acc / (1.0f + expf(-acc));
    if (wr != nullptr) {
      if (f < K) wr[(int64_t)(K - 1 - f) * C + c] = x0;
      if (i == 0)
        for (int e = 0; e < K - n; ++e) wr[(int64_t)e * C + c] = rd[(int64_t)(e + n) * C + c];
    }
  }
  float* o = out + (int64_t)t * C + c0;
  const int first_head = c0 / dim;
  const int unit_here = min(max(n_unit - first_head, 0), nc / dim);   // unit heads of this chunk
  if (unit_here == 0) {                   // every thread re-reads only what it wrote itself
    for (int cc = threadIdx.x; cc < nc; cc += blockDim.x) o[cc] = ys[cc];
    return;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int hd = wid; hd < unit_here; hd += nw) {
    float ss = 0.f;
    for (int e = lane; e < dim; e += 64) {
      const float v = ys[hd * dim + e];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss + unit_eps);
    for (int e = lane; e < dim; e += 64) o[hd * dim + e] = ys[hd * dim + e] * r;
  }
  for (int cc = unit_here * dim + threadIdx.x; cc < nc; cc += blockDim.x) o[cc] = ys[cc];
}

// Four channels per thread (2 to 4 taps; C, dim, the row stride and the chunk multiples of 4,
// 16-byte aligned rows): one 8- or 16-byte load per tap row, the four channels' taps as 4 * taps
// contiguous floats, 16-byte state accesses and stores.
__device__ __forceinline__ float4 ld4any(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4any(const bf16_t* p) {
  const uint2 w = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                     __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
}

template <typename T, int TAPS>
__global__ __launch_bounds__(256) void conv_act_heads_vec_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
    float* __restrict__ state, const int32_t* __restrict__ row_state,
    const int32_t* __restrict__ row_back, const int32_t* __restrict__ row_fwd,
    const int32_t* __restrict__ pos, float* __restrict__ out, int C, int, int slots,
    int n_unit, int dim, float unit_eps, int chunk) {
  constexpr int taps = TAPS;
  extern __shared__ __attribute__((aligned(16))) float ys[];
  const int t = blockIdx.x;
  const int c0 = blockIdx.y * chunk;
  const int nc = min(chunk, C - c0);
  const int code = row_state[t], i = row_back[t], f = row_fwd[t], p = pos[t];
  const int K = taps - 1;
  const float* rd = code >= 0 ? state + ((int64_t)((code & 1) * slots + (code >> 1)) * K) * C : nullptr;
  float* wr = code >= 0 ? state + ((int64_t)((1 - (code & 1)) * slots + (code >> 1)) * K) * C : nullptr;
  const T* xr = x + (int64_t)t * x_stride;
  const int n = i + f + 1;
  for (int cc = threadIdx.x * 4; cc < nc; cc += blockDim.x * 4) {
    const int c = c0 + cc;
    const float4 x0 = ld4any(xr + c);
    float wc[4 * TAPS];                                  // [4][taps], read in 16-byte pieces
#pragma unroll
    for (int k = 0; k < TAPS; ++k)
      *reinterpret_cast<float4*>(wc + 4 * k) = ld4any(w + (int64_t)c * taps + 4 * k);
    float a0 = wc[taps - 1] * x0.x, a1 = wc[2 * taps - 1] * x0.y;
    float a2 = wc[3 * taps - 1] * x0.z, a3 = wc[4 * taps - 1] * x0.w;
#pragma unroll
    for (int dl = 1; dl < taps; ++dl) {
      float4 src;
      if (dl <= i) src = ld4any(xr - (int64_t)dl * x_stride + c);
      else if (p - dl >= 0 && rd != nullptr) src = ld4any(rd + (int64_t)(K + i - dl) * C + c);
      else continue;
      const int k = taps - 1 - dl;
      a0 += wc[k] * src.x;
      a1 += wc[taps + k] * src.y;
      a2 += wc[2 * taps + k] * src.z;
      a3 += wc[3 * taps + k] * src.w;
    }
    *reinterpret_cast<float4*>(ys + cc) =
        make_float4(a0 / (1.0f + expf(-a0)), a1 / (1.0f + expf(-a1)), a2 / (1.0f + expf(-a2)),
                    a3 / (1.0f + expf(-a3)));
    if (wr != nullptr) {
      if (f < K) *reinterpret_cast<float4*>(wr + (int64_t)(K - 1 - f) * C + c) = x0;
      if (i == 0)
        for (int e = 0; e < K - n; ++e)
          *reinterpret_cast<float4*>(wr + (int64_t)e * C + c) = ld4any(rd + (int64_t)(e + n) * C + c);
    }
  }
  float* o = out + (int64_t)t * C + c0;
  const int first_head = c0 / dim;
  const int unit_here = min(max(n_unit - first_head, 0), nc / dim);
  if (unit_here == 0) {                   // every thread re-reads only what it wrote itself
    for (int cc = threadIdx.x * 4; cc < nc; cc += blockDim.x * 4)
      *reinterpret_cast<float4*>(o + cc) = *reinterpret_cast<const float4*>(ys + cc);
    return;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int hd = wid; hd < unit_here; hd += nw) {
    float ss = 0.f;
    for (int e = lane; e < dim; e += 64) {
      const float v = ys[hd * dim + e];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss + unit_eps);
    for (int e = lane; e < dim; e += 64) o[hd * dim + e] = ys[hd * dim + e] * r;
  }
  for (int cc = unit_here * dim + threadIdx.x; cc < nc; cc += blockDim.x) o[cc] = ys[cc];
}

// One thread per row: the `top` largest of z + bias (ties to the lower index), weights =
// softmax over the chosen.  E <= 256.
__global__ __launch_bounds__(64) void moe_route_topk_kernel(
    const float* __restrict__ z, const float* __restrict__ bias, int T_, int E, int top,
    int32_t* __restrict__ ids, float* __restrict__ weights) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T_) return;
  const float* zr = z + (int64_t)t * E;
  int32_t* id = ids + (int64_t)t * top;
  float* wt = weights + (int64_t)t * top;
  float prev = __builtin_huge_valf();
  int prev_i = -1;
  float mx = 0.f;
  for (int k = 0; k < top; ++k) {
    // the largest entry after (prev, prev_i) in the order (value descending, index ascending)
    float best = -__builtin_huge_valf();
    int bi = -1;
    for (int e = 0; e < E; ++e) {
      const float v = zr[e] + (bias != nullptr ? bias[e] : 0.f);
      const bool after = v < prev || (v == prev && e > prev_i);
      if (after && (bi < 0 || v > best)) {
        best = v;
        bi = e;
      }
    }
    if (bi < 0) {                       // non-finite logits: keep the indices valid
      bi = k < E ? k : 0;
      best = -__builtin_huge_valf();
    }
    id[k] = bi;
    wt[k] = best;
    if (k == 0) mx = best;
    prev = best;
    prev_i = bi;
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    const float e = expf(wt[k] - mx);
    wt[k] = e;
    sum += e;
  }
  for (int k = 0; k < top; ++k) wt[k] /= sum;
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_rows_kernel(const T* __restrict__ x, int64_t x_stride,
                                                        T* __restrict__ out, int64_t o_stride,
                                                        int F) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < F; c += gridDim.y * blockDim.x) {
    const float v = ldf(x + (int64_t)t * x_stride + c);
    stf(out + (int64_t)t * o_stride + c, 0.5f * v * (1.0f + erff(v * 0.70710678118654752f)));
  }
}

// ------------------------------------------------------------------ launchers
void launch_residual_add_norm(bool out_f32, float* x, const void* y1, int64_t y1s, bool y1f,
                              const void* y2, int64_t y2s, bool y2f, const float* shift,
                              const float* w, float eps, float offset, void* out, int T_, int d,
                              float mult, hipStream_t s) {
  if (T_ == 0) return;
  if (out_f32)
    hipLaunchKernelGGL(residual_add_norm_kernel<float>, dim3(T_), dim3(256), 0, s, x, y1, y1s, y1f,
                       y2, y2s, y2f, shift, w, eps, offset, (float*)out, d, mult);
  else
    hipLaunchKernelGGL(residual_add_norm_kernel<bf16_t>, dim3(T_), dim3(256), 0, s, x, y1, y1s,
                       y1f, y2, y2s, y2f, shift, w, eps, offset, (bf16_t*)out, d, mult);
}

void launch_rotary_append(bool f32, const void* qkv, int64_t stride, const int32_t* pos,
                          const float* inv_freq, int nrot, const int32_t* slots, void* k_cache,
                          void* v_cache, int T_, int H, int G, int maps, int dim, int vdim, int BS,
                          int64_t pool_slots, float* q_out, hipStream_t s) {
  if (T_ == 0) return;
  const size_t lds = (size_t)(2 * nrot + 2) * sizeof(float);     // dim <= 8192: checked by the caller
  const bool vec = dim % 8 == 0 && vdim % 8 == 0 && stride % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(qkv) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(v_cache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(q_out) % 16 == 0;
#define ROT_GO(KERNEL, TT)                                                                     \
  hipLaunchKernelGGL(KERNEL<TT>, dim3(T_), dim3(256), lds, s, (const TT*)qkv, stride, pos,    \
                     inv_freq, nrot, slots, (TT*)k_cache, (TT*)v_cache, H, G, maps, dim, vdim, \
                     BS, pool_slots, q_out)
  if (vec) {
    if (f32) ROT_GO(rotary_append_vec_kernel, float);
    else ROT_GO(rotary_append_vec_kernel, bf16_t);
  } else {
    if (f32) ROT_GO(rotary_append_kernel, float);
    else ROT_GO(rotary_append_kernel, bf16_t);
  }
#undef ROT_GO
}

void launch_conv_act_heads(bool f32, const void* x, int64_t stride, const float* w, float* state,
                           const int32_t* row_state, const int32_t* row_back,
                           const int32_t* row_fwd, const int32_t* pos, float* out, int T_, int C,
                           int taps, int slots, int n_unit, int dim, float unit_eps,
                           hipStream_t s) {
  if (T_ == 0) return;
  // about 1024 channels per workgroup (four per thread), whole heads; rows of few channels
  // or steps of few rows get smaller chunks so that the grid still fills the chip
  const int want = (T_ >= 1024 && C >= 4096) ? 1024 : 256;
  const int chunk = dim * ((want + dim - 1) / dim);
  const size_t lds = (size_t)chunk * sizeof(float);
  const dim3 grid(T_, (C + chunk - 1) / chunk);
  const bool vec = taps >= 2 && taps <= 4 && C % 4 == 0 && dim % 4 == 0 && stride % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(state) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0;
#define CONV_GO(KERNEL, TT)                                                                     \
  hipLaunchKernelGGL(KERNEL<TT>, grid, dim3(256), lds, s, (const TT*)x, stride, w, state,      \
                     row_state, row_back, row_fwd, pos, out, C, taps, slots, n_unit, dim,       \
                     unit_eps, chunk)
#define CONV_VEC(TT)                                                                            \
  do {                                                                                          \
    if (taps == 2) hipLaunchKernelGGL((conv_act_heads_vec_kernel<TT, 2>), grid, dim3(256), lds, s, (const TT*)x, stride, w, state, row_state, row_back, row_fwd, pos, out, C, taps, slots, n_unit, dim, unit_eps, chunk); \
    else if (taps == 3) hipLaunchKernelGGL((conv_act_heads_vec_kernel<TT, 3>), grid, dim3(256), lds, s, (const TT*)x, stride, w, state, row_state, row_back, row_fwd, pos, out, C, taps, slots, n_unit, dim, unit_eps, chunk); \
    else hipLaunchKernelGGL((conv_act_heads_vec_kernel<TT, 4>), grid, dim3(256), lds, s, (const TT*)x, stride, w, state, row_state, row_back, row_fwd, pos, out, C, taps, slots, n_unit, dim, unit_eps, chunk); \
  } while (0)
  if (vec) {
    if (f32) CONV_VEC(float);
    else CONV_VEC(bf16_t);
  } else {
    if (f32) CONV_GO(conv_act_heads_kernel, float);
    else CONV_GO(conv_act_heads_kernel, bf16_t);
  }
#undef CONV_GO
#undef CONV_VEC
}

void launch_moe_route_topk(const float* z, const float* bias, int T_, int E, int top, int32_t* ids,
                           float* weights, hipStream_t s) {
  if (T_ == 0) return;
  hipLaunchKernelGGL(moe_route_topk_kernel, dim3((T_ + 63) / 64), dim3(64), 0, s, z, bias, T_, E,
                     top, ids, weights);
}

void launch_gelu_rows(bool f32, const void* x, int64_t xs, void* out, int64_t os, int T_, int F,
                      hipStream_t s) {
  if (T_ == 0) return;
  const dim3 grid(T_, (unsigned)((F + 1023) / 1024 > 0 ? (F + 1023) / 1024 : 1));
  if (f32)
    hipLaunchKernelGGL(gelu_rows_kernel<float>, grid, dim3(256), 0, s, (const float*)x, xs,
                       (float*)out, os, F);
  else
    hipLaunchKernelGGL(gelu_rows_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)x, xs,
                       (bf16_t*)out, os, F);
}

}  // namespace rfqmix
