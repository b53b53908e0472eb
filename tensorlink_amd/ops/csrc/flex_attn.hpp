// Options of the flexible paged attention kernels beyond window / sink /
// score cap, shared by the row kernel, the MFMA tile kernel and the
// bindings. Passed by value; every field's zero value switches it off.
#pragma once

struct TlFlexExtra {
  // visibility. Query i sees key j <= i when j >= lo(i) or j < keep, with
  //   lo(i) = i - window + 1          (window > 0, given separately)
  //         = floor(i / chunk) * chunk (chunk > 0: the query's own chunk,
  //                                     counted from position 0)
  //         = 0                        otherwise
  int chunk;
  int keep;
  // learned distance bias added to the scaled score (not scaled itself):
  // bias[h * nb + min(i - j, nb - 1)], fp32 [H][nb]; null = none
  const float* bias;
  int nb;
  // output gate: the attended row of head h is multiplied by
  // sigmoid(gate[t * gate_ld + gate_col + (gate_heads ? h : h * V + c)]);
  // pre-activations in fp32 or bf16 (gate_f32); null = none
  const void* gate;
  int gate_ld, gate_col, gate_heads, gate_f32;
};

// first visible position of the main key range of a query at `pos`
__host__ __device__ inline int tl_flex_lo(int pos, int window, int chunk) {
  if (window > 0) return pos - window + 1 > 0 ? pos - window + 1 : 0;
  if (chunk > 0) return (pos / chunk) * chunk;
  return 0;
}
