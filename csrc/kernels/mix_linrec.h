// Arguments of the gated linear recurrence's launcher (mix_linrec.hip), shared with the
// bindings.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfqmix {

struct LinrecArgs {
  const void *q, *k, *v;            // [T, Hq, dim] x2, [T, H, vdim]; row strides below
  int64_t qs, ks, vs;
  const float* z;                   // decay logits [T, H dim] (decay_ready: the decays themselves)
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
  int decay_ready;
  float* raw;                       // [T, H vdim] fp32 scratch or null: read-outs before norm and gate
  float* state;                     // [2 slots, H, dim, vdim]
  const int32_t *row_state, *row_back, *row_fwd, *pos, *run_rows;
  int runs;
  void* out;                        // [T, H vdim]
  int T, H, rep, dim, vdim, slots;
};

bool linrec_ok(int dim, int vdim);
void launch_decay_from_logits(float* z, int64_t z_stride, const float* rate, const float* zbias,
                              float zsign, int T, int H, int dim, hipStream_t s);
void launch_gated_linrec(bool in_f32, bool act_f32, bool delta, const LinrecArgs& a, hipStream_t s);

}  // namespace rfqmix
