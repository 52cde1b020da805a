// Gated linear recurrences with a decay per key channel, plain or with the delta rule.
//
// Per head a state S of dim key x vdim value channels (fp32), token by token inside a run:
//
//   a_t = exp(-rate_h softplus(zsign (z_t + zbias)))       decay per key channel
//   S  <- diag(a_t) S
//   u_t = beta_t (v_t - S^T k_t)          delta rule (beta_t = sigmoid of a logit per head);
//                                          without it u_t = v_t
//   S  <- S + k_t u_t^T ;  o_t = q_scale S^T q_t           the read-out sees the token's write
//   out_t = o_t / sqrt(mean(o_t^2) + eps) * norm_w * act(gate_t)    act = silu or sigmoid
//
// sigmoid(z)^(1 / tau) is the case zsign = -1, rate = 1 / tau; exp(-A softplus(z + b)) the
// case zsign = +1, rate = A.  Query and key heads may be shared by several value heads.
//
// Rows of a sequence are contiguous in a step (a "run").  row_state = slot * 2 + half to read
// (-1: none), row_back = index of the row inside its run, row_fwd = rows of the run after it.
// The state pool is double buffered: a run reads its sequence's half and writes the other, and
// a run that starts at position 0 reads nothing (the slot may hold another sequence's rest).
//
// One workgroup per (run, head); thread j owns value channel j: column j of S lives in
// registers when dim is a compile-time size, else in LDS.  q, k and the decay of a token reach
// all threads through LDS (one 16-byte read per key channel); the next token's operands are
// loaded while the current one is summed.
#include "mix_common.h"
#include "mix_linrec.h"

namespace rfqmix {

__device__ __forceinline__ float softplus_f(float y) {
  return fmaxf(y, 0.f) + log1pf(expf(-fabsf(y)));
}

template <typename TI, typename TG, int NR, bool DELTA>
__global__ __launch_bounds__(256) void gated_linrec_kernel(
    const TI* __restrict__ q, const TI* __restrict__ k, const TI* __restrict__ v,
    int64_t q_stride, int64_t k_stride, int64_t v_stride, const float* __restrict__ z,
    int64_t z_stride, const float* __restrict__ rate, const float* __restrict__ zbias,
    float zsign, const TG* __restrict__ beta, int64_t b_stride, const TG* __restrict__ gate,
    int64_t g_stride, int gate_sigmoid, const float* __restrict__ norm_w, float eps,
    float q_scale, int decay_ready, float* __restrict__ raw, float* __restrict__ state,
    const int32_t* __restrict__ row_state,
    const int32_t* __restrict__ row_back, const int32_t* __restrict__ row_fwd,
    const int32_t* __restrict__ pos, const int32_t* __restrict__ run_rows, TG* __restrict__ out,
    int H, int rep, int dim, int vdim, int slots) {
  const int t0 = run_rows != nullptr ? run_rows[blockIdx.x] : (int)blockIdx.x;
  const int h = blockIdx.y;
  if (t0 < 0 || row_back[t0] != 0) return;
  const int n = row_fwd[t0] + 1;
  const int code = row_state[t0];
  const int j = threadIdx.x;
  const bool vlive = j < vdim, klive = j < dim;
  const int hq = h / rep;
  const int qc = hq * dim + (klive ? j : 0);           // this thread's query / key channel
  const int zc = h * dim + (klive ? j : 0);            // its decay channel
  const int vc = h * vdim + (vlive ? j : 0);           // its value / gate / output channel

  extern __shared__ __attribute__((aligned(16))) float lds[];
  float4* ops = reinterpret_cast<float4*>(lds);        // [2][dim] of (q, k, decay, -)
  float* scratch = lds + 8 * dim;                      // 16
  float* st = scratch + 16;                            // [dim][vdim] when NR == 0
  float sreg[NR > 0 ? NR : 1];

  const bool from_state = code >= 0 && pos[t0] > 0;
  const int64_t hsz = (int64_t)dim * vdim;
  const float* rd = state + (((int64_t)(code & 1) * slots + (code >> 1)) * H + h) * hsz;
  if (NR > 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i) sreg[i] = (from_state && vlive) ? rd[i * vdim + j] : 0.f;
  } else if (vlive) {
    for (int i = 0; i < dim; ++i) st[i * vdim + j] = from_state ? rd[i * vdim + j] : 0.f;
  }

  const float my_rate = rate[h];
  const float my_zb = klive ? zbias[zc] : 0.f;
  const float my_nw = vlive ? norm_w[j] : 0.f;
  float nq = 0.f, nk = 0.f, na = 0.f, nv = 0.f, ng = 0.f, nb = 0.f;
  if (klive) {
    nq = ldf(q + (int64_t)t0 * q_stride + qc);
    nk = ldf(k + (int64_t)t0 * k_stride + qc);
    na = z[(int64_t)t0 * z_stride + zc];
    if (!decay_ready) na = expf(-my_rate * softplus_f(zsign * (na + my_zb)));
  }
  if (vlive) {
    nv = ldf(v + (int64_t)t0 * v_stride + vc);
    ng = ldf(gate + (int64_t)t0 * g_stride + vc);
  }
  if (DELTA) nb = ldf(beta + (int64_t)t0 * b_stride + h);

  for (int a = 0; a < n; ++a) {
    const float4* cur = ops + (a & 1) * dim;
    if (klive) ops[(a & 1) * dim + j] = make_float4(nq, nk, na, 0.f);
    const float vj = nv, gj = ng;
    const float bj = DELTA ? 1.0f / (1.0f + expf(-nb)) : 1.f;
    __syncthreads();
    if (a + 1 < n) {                   // the next token's operands, in flight during the sums
      const int64_t t = t0 + a + 1;
      if (klive) {
        nq = ldf(q + t * q_stride + qc);
        nk = ldf(k + t * k_stride + qc);
        na = z[t * z_stride + zc];
      }
      if (vlive) {
        nv = ldf(v + t * v_stride + vc);
        ng = ldf(gate + t * g_stride + vc);
      }
      if (DELTA) nb = ldf(beta + t * b_stride + h);
    }
    float o = 0.f;
    if (vlive) {
      if (DELTA) {
        float acc = 0.f;
        if (NR > 0) {
          float pa[4] = {0.f, 0.f, 0.f, 0.f};      // independent chains: one wave runs per SIMD
#pragma unroll
          for (int i = 0; i < NR; ++i) {
            const float4 c4 = cur[i];
            sreg[i] *= c4.z;
            pa[i & 3] += sreg[i] * c4.y;
          }
          acc = (pa[0] + pa[1]) + (pa[2] + pa[3]);
        } else {
          for (int i = 0; i < dim; ++i) {
            const float4 c4 = cur[i];
            const float s = st[i * vdim + j] * c4.z;
            st[i * vdim + j] = s;
            acc += s * c4.y;
          }
        }
        const float u = bj * (vj - acc);
        if (NR > 0) {
          float po[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NR; ++i) {
            const float4 c4 = cur[i];
            sreg[i] += c4.y * u;
            po[i & 3] += sreg[i] * c4.x;
          }
          o = (po[0] + po[1]) + (po[2] + po[3]);
        } else {
          for (int i = 0; i < dim; ++i) {
            const float4 c4 = cur[i];
            const float s = st[i * vdim + j] + c4.y * u;
            st[i * vdim + j] = s;
            o += s * c4.x;
          }
        }
      } else {
        if (NR > 0) {
          float po[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NR; ++i) {
            const float4 c4 = cur[i];
            sreg[i] = c4.z * sreg[i] + c4.y * vj;
            po[i & 3] += sreg[i] * c4.x;
          }
          o = (po[0] + po[1]) + (po[2] + po[3]);
        } else {
          for (int i = 0; i < dim; ++i) {
            const float4 c4 = cur[i];
            const float s = c4.z * st[i * vdim + j] + c4.y * vj;
            st[i * vdim + j] = s;
            o += s * c4.x;
          }
        }
      }
      o *= q_scale;
    }
    if (a + 1 < n && klive && !decay_ready) na = expf(-my_rate * softplus_f(zsign * (na + my_zb)));
    if (raw != nullptr) {              // long steps: norm and gate follow in a row-parallel kernel
      if (vlive) raw[(int64_t)(t0 + a) * H * vdim + vc] = o;
      continue;
    }
    const float ss = block_sum(vlive ? o * o : 0.f, scratch);
    if (vlive) {
      const float act = gate_sigmoid ? 1.0f / (1.0f + expf(-gj)) : gj / (1.0f + expf(-gj));
      stf(out + (int64_t)(t0 + a) * H * vdim + vc, o / sqrtf(ss / (float)vdim + eps) * my_nw * act);
    }
  }
  if (code >= 0 && vlive) {
    float* wr = state + (((int64_t)(1 - (code & 1)) * slots + (code >> 1)) * H + h) * hsz;
    if (NR > 0) {
#pragma unroll
      for (int i = 0; i < NR; ++i) wr[i * vdim + j] = sreg[i];
    } else {
      for (int i = 0; i < dim; ++i) wr[i * vdim + j] = st[i * vdim + j];
    }
  }
}

// z[t, h, c] <- exp(-rate_h softplus(zsign (z + zbias[h, c]))) in place: the decays of a long
// step are formed by all threads of the chip at once instead of inside the token-by-token scan.
__global__ __launch_bounds__(256) void decay_from_logits_kernel(
    float* __restrict__ z, int64_t z_stride, const float* __restrict__ rate,
    const float* __restrict__ zbias, float zsign, int HD, int dim) {
  const int t = blockIdx.x;
  float* zr = z + (int64_t)t * z_stride;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < HD; c += gridDim.y * blockDim.x)
    zr[c] = expf(-rate[c / dim] * softplus_f(zsign * (zr[c] + zbias[c])));
}

void launch_decay_from_logits(float* z, int64_t z_stride, const float* rate, const float* zbias,
                              float zsign, int T, int H, int dim, hipStream_t s) {
  if (T == 0) return;
  const int HD = H * dim;
  hipLaunchKernelGGL(decay_from_logits_kernel, dim3(T, (HD + 1023) / 1024), dim3(256), 0, s, z,
                     z_stride, rate, zbias, zsign, HD, dim);
}

// out[t, h, :] = raw / sqrt(mean(raw^2) + eps) * norm_w * act(gate): the scan's read-outs of a
// long step, a wave per (row, head).
template <typename TG>
__global__ __launch_bounds__(256) void linrec_finish_kernel(
    const float* __restrict__ raw, const TG* __restrict__ gate, int64_t g_stride,
    int gate_sigmoid, const float* __restrict__ norm_w, float eps, TG* __restrict__ out, int T,
    int H, int vdim) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= (int64_t)T * H) return;
  const int64_t t = item / H;
  const int h = (int)(item - t * H);
  const float* r = raw + item * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += 64) ss += r[c] * r[c];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int c = lane; c < vdim; c += 64) {
    const float gj = ldf(gate + t * g_stride + (int64_t)h * vdim + c);
    const float act = gate_sigmoid ? 1.0f / (1.0f + expf(-gj)) : gj / (1.0f + expf(-gj));
    stf(out + item * vdim + c, r[c] * inv * norm_w[c] * act);
  }
}

// The scan of a long step: decays formed ahead (z holds them), read-outs to `raw` for the
// row-parallel norm and gate.  One WAVE per (run, head, 64 value channels), no LDS and no
// barrier: every wave loads the token's q, k and decay itself, a key channel per lane (two for
// dim 128), and broadcasts channel i to all lanes with v_readlane, so the sums run on scalar
// operands; the next token's operands are loaded while the current one is summed.
template <typename TI, typename TG, int NR, bool DELTA>
__global__ __launch_bounds__(64) void gated_linrec_scan_kernel(
    const TI* __restrict__ q, const TI* __restrict__ k, const TI* __restrict__ v,
    int64_t q_stride, int64_t k_stride, int64_t v_stride, const float* __restrict__ z,
    int64_t z_stride, const TG* __restrict__ beta, int64_t b_stride, float q_scale,
    float* __restrict__ raw, float* __restrict__ state, const int32_t* __restrict__ row_state,
    const int32_t* __restrict__ row_back, const int32_t* __restrict__ row_fwd,
    const int32_t* __restrict__ pos, const int32_t* __restrict__ run_rows, int H, int rep,
    int vdim, int slots) {
  constexpr int dim = NR, C = (NR + 63) / 64;
  const int t0 = run_rows != nullptr ? run_rows[blockIdx.x] : (int)blockIdx.x;
  const int h = blockIdx.y;
  if (t0 < 0 || row_back[t0] != 0) return;
  const int n = row_fwd[t0] + 1;
  const int code = row_state[t0];
  const int lane = threadIdx.x;
  const int j = blockIdx.z * 64 + lane;                // this lane's value channel
  const bool vlive = j < vdim;
  const int hq = h / rep;
  const int vc = h * vdim + (vlive ? j : 0);

  float sreg[NR];
  const bool from_state = code >= 0 && pos[t0] > 0;
  const int64_t hsz = (int64_t)dim * vdim;
  const float* rd = state + (((int64_t)(code & 1) * slots + (code >> 1)) * H + h) * hsz;
#pragma unroll
  for (int i = 0; i < NR; ++i) sreg[i] = (from_state && vlive) ? rd[i * vdim + j] : 0.f;

  float nq[C], nk[C], na[C], nv = 0.f, nb = 0.f;
  auto load = [&](int64_t t) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int ch = c * 64 + lane;
      const bool ok = ch < dim;
      nq[c] = ok ? ldf(q + t * q_stride + hq * dim + ch) : 0.f;
      nk[c] = ok ? ldf(k + t * k_stride + hq * dim + ch) : 0.f;
      na[c] = ok ? z[t * z_stride + h * dim + ch] : 0.f;
    }
    if (vlive) nv = ldf(v + t * v_stride + vc);
    if (DELTA) nb = ldf(beta + t * b_stride + h);
  };
  load(t0);
  for (int a = 0; a < n; ++a) {
    int cq[C], ck[C], ca[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      cq[c] = __float_as_int(nq[c]);
      ck[c] = __float_as_int(nk[c]);
      ca[c] = __float_as_int(na[c]);
    }
    const float vj = nv;
    const float bj = DELTA ? 1.0f / (1.0f + expf(-nb)) : 1.f;
    if (a + 1 < n) load(t0 + a + 1);
    float po[4] = {0.f, 0.f, 0.f, 0.f};
    if (DELTA) {
      float pa[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const float ai = __int_as_float(__builtin_amdgcn_readlane(ca[i >> 6], i & 63));
        const float ki = __int_as_float(__builtin_amdgcn_readlane(ck[i >> 6], i & 63));
        sreg[i] *= ai;
        pa[i & 3] += sreg[i] * ki;
      }
      const float u = bj * (vj - ((pa[0] + pa[1]) + (pa[2] + pa[3])));
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const float ki = __int_as_float(__builtin_amdgcn_readlane(ck[i >> 6], i & 63));
        const float qi = __int_as_float(__builtin_amdgcn_readlane(cq[i >> 6], i & 63));
        sreg[i] += ki * u;
        po[i & 3] += sreg[i] * qi;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const float ai = __int_as_float(__builtin_amdgcn_readlane(ca[i >> 6], i & 63));
        const float ki = __int_as_float(__builtin_amdgcn_readlane(ck[i >> 6], i & 63));
        const float qi = __int_as_float(__builtin_amdgcn_readlane(cq[i >> 6], i & 63));
        sreg[i] = ai * sreg[i] + ki * vj;
        po[i & 3] += sreg[i] * qi;
      }
    }
    if (vlive) raw[(int64_t)(t0 + a) * H * vdim + vc] = ((po[0] + po[1]) + (po[2] + po[3])) * q_scale;
  }
  if (code >= 0 && vlive) {
    float* wr = state + (((int64_t)(1 - (code & 1)) * slots + (code >> 1)) * H + h) * hsz;
#pragma unroll
    for (int i = 0; i < NR; ++i) wr[i * vdim + j] = sreg[i];
  }
}

// ------------------------------------------------------------------ launchers
template <typename TI, typename TG, int NR, bool DELTA>
static void launch_linrec_one(const LinrecArgs& a, hipStream_t s) {
  if constexpr (NR > 0) {
    if (a.raw != nullptr && a.decay_ready) {
      const dim3 grid(a.run_rows != nullptr ? a.runs : a.T, a.H, (a.vdim + 63) / 64);
      hipLaunchKernelGGL((gated_linrec_scan_kernel<TI, TG, NR, DELTA>), grid, dim3(64), 0, s,
                         (const TI*)a.q, (const TI*)a.k, (const TI*)a.v, a.qs, a.ks, a.vs, a.z, a.zs,
                         (const TG*)a.beta, a.bs, a.q_scale, a.raw, a.state, a.row_state,
                         a.row_back, a.row_fwd, a.pos, a.run_rows, a.H, a.rep, a.vdim, a.slots);
      return;
    }
  }
  const int threads = ((a.dim > a.vdim ? a.dim : a.vdim) + 63) / 64 * 64;
  const size_t lds = (size_t)(8 * a.dim + 16 + (NR > 0 ? 0 : a.dim * a.vdim)) * 4;
  static bool attr = false;
  if (!attr) {          // dynamic LDS above 64 KB has to be allowed per kernel, once
    hipFuncSetAttribute(reinterpret_cast<const void*>(&gated_linrec_kernel<TI, TG, NR, DELTA>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    attr = true;
  }
  hipLaunchKernelGGL((gated_linrec_kernel<TI, TG, NR, DELTA>),
                     dim3(a.run_rows != nullptr ? a.runs : a.T, a.H), dim3(threads), lds, s,
                     (const TI*)a.q, (const TI*)a.k, (const TI*)a.v, a.qs, a.ks, a.vs, a.z, a.zs,
                     a.rate, a.zbias, a.zsign, (const TG*)a.beta, a.bs, (const TG*)a.gate, a.gs,
                     a.gate_sigmoid, a.norm_w, a.eps, a.q_scale, a.decay_ready, a.raw, a.state,
                     a.row_state, a.row_back,
                     a.row_fwd, a.pos, a.run_rows, (TG*)a.out, a.H, a.rep, a.dim, a.vdim, a.slots);
}

template <typename TI, typename TG, bool DELTA>
static void launch_linrec_dim(const LinrecArgs& a, hipStream_t s) {
  if (a.dim == 32) launch_linrec_one<TI, TG, 32, DELTA>(a, s);
  else if (a.dim == 64) launch_linrec_one<TI, TG, 64, DELTA>(a, s);
  else if (a.dim == 128) launch_linrec_one<TI, TG, 128, DELTA>(a, s);
  else launch_linrec_one<TI, TG, 0, DELTA>(a, s);
}

// Whether the head sizes fit (threads <= 256; a head's state in registers or LDS).
bool linrec_ok(int dim, int vdim) {
  if (dim < 1 || vdim < 1 || dim > 256 || vdim > 256) return false;
  if (dim == 32 || dim == 64 || dim == 128) return true;
  return (size_t)(8 * dim + 16 + dim * vdim) * 4 <= (size_t)160 * 1024;
}

// in_f32: q, k, v are fp32 (else bf16); act_f32: beta, gate and out are fp32 (else bf16).
void launch_gated_linrec(bool in_f32, bool act_f32, bool delta, const LinrecArgs& a,
                         hipStream_t s) {
  if (a.T == 0 || (a.run_rows != nullptr && a.runs == 0)) return;
#define LINREC_GO(TI, TG)                                   \
  do {                                                      \
    if (delta) launch_linrec_dim<TI, TG, true>(a, s);       \
    else launch_linrec_dim<TI, TG, false>(a, s);            \
  } while (0)
  if (in_f32 && act_f32) LINREC_GO(float, float);
  else if (in_f32) LINREC_GO(float, bf16_t);
  else if (!act_f32) LINREC_GO(bf16_t, bf16_t);
  else LINREC_GO(bf16_t, float);
#undef LINREC_GO
  if (a.raw != nullptr) {
    const int64_t items = (int64_t)a.T * a.H;
    const dim3 grid((unsigned)((items + 3) / 4));
    if (act_f32)
      hipLaunchKernelGGL(linrec_finish_kernel<float>, grid, dim3(256), 0, s, a.raw,
                         (const float*)a.gate, a.gs, a.gate_sigmoid, a.norm_w, a.eps,
                         (float*)a.out, a.T, a.H, a.vdim);
    else
      hipLaunchKernelGGL(linrec_finish_kernel<bf16_t>, grid, dim3(256), 0, s, a.raw,
                         (const bf16_t*)a.gate, a.gs, a.gate_sigmoid, a.norm_w, a.eps,
                         (bf16_t*)a.out, a.T, a.H, a.vdim);
  }
}

}  // namespace rfqmix
