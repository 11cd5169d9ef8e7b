// Arguments of the column scans (csrc/mixers/column_scan.hip), shared with the torch bindings.
#pragma once

namespace mxs {

struct ScanArgs {
  float* out;          // [T, H*dv]
  const void* q;       // delta rule: queries [T, G*dk]; state space: C [T, G*dk]
  long q_stride;
  const void* k;       // delta rule: keys; state space: B
  long k_stride;
  const void* v;       // delta rule: values [T, H*dv]; state space: x
  long v_stride;
  const void* beta;    // delta rule: write strength before the sigmoid [T, H]; state space: dt before the softplus [T, H]
  long beta_stride;
  const void* a;       // delta rule: decay pre-activation [T, H*dk]
  long a_stride;
  const float* dt_bias;  // delta rule: [H*dk]; state space: [H]
  const float* A_log;    // [H]
  const float* D;        // state space: [H]
  float* state;          // [slots, state_stride], this layer's S at `off` as [H][dv][dk]
  long state_stride;
  const int* state_rows;
  long off;
  const int* qsl;
  const int* seq_lens;
  int n_rows, H, G, dk, dv;
  int max_q;  // the step's longest chunk; 1: single tokens only (a smaller stage)
  float q_scale, unit_eps;
  // state space, long chunks cut into pieces that run side by side: mode 0 whole chunk, state from and
  // to the slot; mode 1 a piece from an empty state, its end state to sc_local and its summed decay
  // exponents to sc_decay, no outputs; mode 2 a piece from sc_start, outputs, the sequence's last
  // piece writes the slot
  int mode, piece, npieces;
  float* sc_local;   // [S, npieces, H*dv*dk]
  float* sc_start;   // [S, npieces, H*dv*dk]
  float* sc_decay;   // [S, npieces, H]
};

}  // namespace mxs
