// Arguments of the gated linear recurrence's launcher (mix_linrec.hip), shared with the
// bindings.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfqmix {

struct LinrecArgs {
  const void *q, *k, *v;            // [T, Hq, dim] x2, [T, H, vdim]; row strides below
  int64_t qs, ks, vs;
  const float* z;                   // decay logits [T, H dim]
  int64_t zs;
  const float *rate, *zbias;        // [H], [H dim]
  float zsign;
  const void* beta;                 // [T, H] logits (delta rule) or null
  int64_t bs;
  const void* gate;                 // [T, H vdim]
  int64_t gs;
  int gate_sigmoid;
  const float* norm_w;              // [vdim]
  float eps, q_scale;
  float* state;                     // [2 slots, H, dim, vdim]
  const int32_t *row_state, *row_back, *row_fwd, *pos, *run_rows;
  int runs;
  void* out;                        // [T, H vdim]
  int T, H, rep, dim, vdim, slots;
};

bool linrec_ok(int dim, int vdim);
void launch_gated_linrec(bool in_f32, bool act_f32, bool delta, const LinrecArgs& a, hipStream_t s);

}  // namespace rfqmix
