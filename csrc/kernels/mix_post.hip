// Row kernels of post-norm residual layers: embedding rows into the fp32 stream, the
// residual update x += m * rms(y) (1 + w) with a copy of the stream in the activation type,
// RMS norms of (column slices of) projection outputs, the latent norm with its paged-cache
// append, SwiGLU, and the logit soft cap.
//
// One workgroup per token row; norms and the residual stream are fp32 whatever the
// activation type is.
#include "mix_common.h"

namespace rfqmix {

template <typename T>
__global__ __launch_bounds__(256) void embed_rows_kernel(
    const int32_t* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out, int d,
    int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (int64_t)id * d;
  float* o = out + (int64_t)t * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x) o[c] = ldf(row + c) * scale;
}

// residual[t] += mult * y[t] / sqrt(mean(y[t]^2) + eps) * (1 + w); copy (nullable) receives
// the updated row rounded to bf16.
template <typename TY>
__global__ __launch_bounds__(256) void post_norm_add_kernel(
    const TY* __restrict__ y, int64_t y_stride, float* __restrict__ residual,
    const float* __restrict__ w, float mult, float eps, bf16_t* __restrict__ copy, int d) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const TY* yr = y + (int64_t)t * y_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float v = ldf(yr + c);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = mult / sqrtf(ss / (float)d + eps);
  float* x = residual + (int64_t)t * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float v = x[c] + ldf(yr + c) * r * (1.0f + w[c]);
    x[c] = v;
    if (copy != nullptr) stf(copy + (int64_t)t * d + c, v);
  }
}

// out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * (w + offset); x rows have a stride.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(
    const TI* __restrict__ x, int64_t x_stride, const float* __restrict__ w, float eps,
    float offset, TO* __restrict__ out, int n) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const TI* xr = x + (int64_t)t * x_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = ldf(xr + c);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    stf(out + (int64_t)t * n + c, ldf(xr + c) * r * (w[c] + offset));
}

// c[t] = rms(x[t]) * w into pool[slot / BS, 0, slot % BS, :] (pool [blocks, 1, BS, R]).
template <typename T>
__global__ __launch_bounds__(256) void latent_norm_append_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, float eps,
    const int32_t* __restrict__ slots, T* __restrict__ pool, int R, int64_t pool_rows) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int32_t slot = slots[t];
  if (slot < 0 || slot >= pool_rows) return;           // uniform per workgroup
  const T* xr = x + (int64_t)t * x_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += blockDim.x) {
    const float v = ldf(xr + c);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)R + eps);
  T* o = pool + (int64_t)slot * R;
  for (int c = threadIdx.x; c < R; c += blockDim.x) stf(o + c, ldf(xr + c) * r * w[c]);
}

// out[t, f] = silu(gu[t, f]) * gu[t, F + f]
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_any_kernel(
    const T* __restrict__ gu, int64_t gu_stride, T* __restrict__ out, int F, int64_t total) {
  for (int64_t x = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; x < total;
       x += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = x / F;
    const int f = (int)(x - t * F);
    const float g = ldf(gu + t * gu_stride + f), u = ldf(gu + t * gu_stride + F + f);
    stf(out + x, g / (1.0f + expf(-g)) * u);
  }
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, float cap, float inv,
                                                      int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv);
}

// ------------------------------------------------------------------ launchers
void launch_embed_rows(bool f32, const int32_t* ids, const void* table, float* out, int T, int d,
                       int vocab, float scale, hipStream_t s) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(T), dim3(256), 0, s, ids,
                       (const float*)table, out, d, vocab, scale);
  else
    hipLaunchKernelGGL(embed_rows_kernel<bf16_t>, dim3(T), dim3(256), 0, s, ids,
                       (const bf16_t*)table, out, d, vocab, scale);
}

void launch_post_norm_add(bool y_f32, const void* y, int64_t y_stride, float* residual,
                          const float* w, float mult, float eps, void* copy, int T, int d,
                          hipStream_t s) {
  if (T == 0) return;
  if (y_f32)
    hipLaunchKernelGGL(post_norm_add_kernel<float>, dim3(T), dim3(256), 0, s, (const float*)y,
                       y_stride, residual, w, mult, eps, (bf16_t*)copy, d);
  else
    hipLaunchKernelGGL(post_norm_add_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const bf16_t*)y,
                       y_stride, residual, w, mult, eps, (bf16_t*)copy, d);
}

void launch_rms_norm_rows(bool in_f32, bool out_f32, const void* x, int64_t x_stride,
                          const float* w, float eps, float offset, void* out, int T, int n,
                          hipStream_t s) {
  if (T == 0) return;
  if (in_f32 && out_f32)
    hipLaunchKernelGGL((rms_norm_rows_kernel<float, float>), dim3(T), dim3(256), 0, s,
                       (const float*)x, x_stride, w, eps, offset, (float*)out, n);
  else if (in_f32)
    hipLaunchKernelGGL((rms_norm_rows_kernel<float, bf16_t>), dim3(T), dim3(256), 0, s,
                       (const float*)x, x_stride, w, eps, offset, (bf16_t*)out, n);
  else if (out_f32)
    hipLaunchKernelGGL((rms_norm_rows_kernel<bf16_t, float>), dim3(T), dim3(256), 0, s,
                       (const bf16_t*)x, x_stride, w, eps, offset, (float*)out, n);
  else
    hipLaunchKernelGGL((rms_norm_rows_kernel<bf16_t, bf16_t>), dim3(T), dim3(256), 0, s,
                       (const bf16_t*)x, x_stride, w, eps, offset, (bf16_t*)out, n);
}

void launch_latent_norm_append(bool f32, const void* x, int64_t x_stride, const float* w,
                               float eps, const int32_t* slots, void* pool, int T, int R,
                               int64_t pool_rows, hipStream_t s) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL(latent_norm_append_kernel<float>, dim3(T), dim3(256), 0, s,
                       (const float*)x, x_stride, w, eps, slots, (float*)pool, R, pool_rows);
  else
    hipLaunchKernelGGL(latent_norm_append_kernel<bf16_t>, dim3(T), dim3(256), 0, s,
                       (const bf16_t*)x, x_stride, w, eps, slots, (bf16_t*)pool, R, pool_rows);
}

void launch_silu_mul_any(bool f32, const void* gu, int64_t gu_stride, void* out, int T, int F,
                         hipStream_t s) {
  const int64_t total = (int64_t)T * F;
  if (total == 0) return;
  const int grid = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  if (f32)
    hipLaunchKernelGGL(silu_mul_any_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)gu,
                       gu_stride, (float*)out, F, total);
  else
    hipLaunchKernelGGL(silu_mul_any_kernel<bf16_t>, dim3(grid), dim3(256), 0, s,
                       (const bf16_t*)gu, gu_stride, (bf16_t*)out, F, total);
}

void launch_softcap(float* x, float cap, int64_t total, hipStream_t s) {
  if (total == 0) return;
  const int grid = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  hipLaunchKernelGGL(softcap_kernel, dim3(grid), dim3(256), 0, s, x, cap, 1.0f / cap, total);
}

}  // namespace rfqmix
