// Token-by-token recurrences with a matrix state per head (gfx950): decayed linear attention and
// the mLSTM memory.  The state S [dk, dv] of one (sequence, head) is split over workgroups by
// 64-column slices (columns never interact) and inside a workgroup over 4 waves by rows: thread
// (r, j) keeps rows r*DR .. r*DR+DR-1 of column j in registers for the whole chunk, so a step is
// DR fused multiply-adds for the update, DR for the read-out, and one 4-way sum through LDS.
// Tokens are staged 16 at a time (q, k rows and the v slice as fp32 in LDS, activations applied),
// two barriers per 16 tokens.  The sum order of a token's output does not depend on where a chunk
// starts or ends, so cutting a prompt differently gives the same bits.
// State, decays, gates and every product are fp32; q, k, v come as bf16 or fp32.
//
// Long prompt chunks are also split over time (launch_matrix_scan_split): a sequence's rows are cut
// into pieces of `piece` tokens; pass 1 runs every piece from an empty state and keeps only its end
// state (mLSTM: scaled by its own running maximum, with the piece's summed log forget gates);
// a small kernel chains the pieces' end states into the true state at every piece's start; pass 2
// runs every piece again from that state and writes the outputs.  1.5x the multiply-adds, but as
// many workgroups as pieces instead of one serial walk per (sequence, head, column slice).
#include "mix_common.h"

namespace mxs {

constexpr int kTB = 16;  // tokens per LDS stage

template <typename T, int DR, bool MLSTM>
__global__ void __launch_bounds__(256) matrix_scan_kernel(
    float* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride, const float* __restrict__ decay, const float* __restrict__ gates,
    float* __restrict__ state, long state_stride, const int* __restrict__ state_rows, long off,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, int n_rows, int H, int dk, int dv, int silu,
    float gate_cap, float q_scale, int piece, int npieces, int mode, float* __restrict__ sc_local,
    float* __restrict__ sc_start, long sc_floats) {
  // mode 0: whole chunk, state from and to the slot.  mode 1 (pass 1): piece from an empty state, end
  // state to sc_local, no outputs.  mode 2 (pass 2): piece from sc_start, outputs; the sequence's
  // last piece writes the slot.
  constexpr int DT = 4 * DR;  // padded key size
  __shared__ float sk[kTB][DT];
  __shared__ float sq[kTB][DT];
  __shared__ float sv[kTB][64];
  __shared__ float red[kTB][4][64];
  __shared__ float redn[kTB][4];
  __shared__ float sfa[kTB], sia[kTB], sem[kTB];
  const int s = blockIdx.x / npieces, pc = blockIdx.x - s * npieces, hd = blockIdx.y, c0 = blockIdx.z * 64;
  const int tid = threadIdx.x, j = tid & 63, r = tid >> 6;
  const int row0 = qsl[s];
  if (row0 < 0 || row0 >= n_rows) return;
  const int qlen_all = min(qsl[s + 1], n_rows) - row0;  // never past the step's rows, whatever the metadata says
  const int tb = mode == 0 ? 0 : pc * piece;         // this workgroup's rows of the chunk: [tb, te)
  const int te = mode == 0 ? qlen_all : min(qlen_all, tb + piece);
  if (te <= tb) return;
  const int qlen = te;
  const bool last_piece = te == qlen_all;
  const bool fresh = mode == 1 || (mode == 0 && seq_lens[s] - qlen_all == 0);  // zero state to start from
  const int col = c0 + j;
  const bool col_ok = col < dv;
  float* slot = state + static_cast<long>(state_rows[s]) * state_stride + off;
  const long sc_at = (static_cast<long>(s) * npieces + pc) * sc_floats;
  // where the state comes from and where it goes
  float* src = mode == 2 ? sc_start + sc_at : slot;
  float* dst = mode == 1 ? sc_local + sc_at : slot;
  const bool write_state = mode != 2 || last_piece;
  const long oS = static_cast<long>(hd) * dk * dv, oN = static_cast<long>(H) * dk * dv + static_cast<long>(hd) * dk,
             oM = static_cast<long>(H) * dk * dv + static_cast<long>(H) * dk + hd;
  const float* Sg = src + oS;
  const float* ng = src + oN;
  const float* mg = src + oM;
  float S[DR], nvec[DR];
#pragma unroll
  for (int i = 0; i < DR; ++i) {
    const int d = r * DR + i;
    S[i] = (!fresh && d < dk && col_ok) ? Sg[static_cast<long>(d) * dv + col] : 0.f;
    nvec[i] = (MLSTM && !fresh && d < dk) ? ng[d] : 0.f;
  }
  float m = (MLSTM && !fresh) ? *mg : (mode == 1 ? -INFINITY : 0.f);  // used by thread 0 only
  float fsum = 0.f;                                                    // pass 1: the piece's summed log forget gates
  const float a = MLSTM ? 0.f : decay[hd];
  const int HV = H * dv;
  for (int t0 = tb; t0 < qlen; t0 += kTB) {
    const int nt = min(kTB, qlen - t0);
    __syncthreads();  // the previous stage's reads are done
    for (int idx = tid; idx < nt * DT; idx += 256) {
      const int tt = idx / DT, d = idx - tt * DT;
      float kv = 0.f, qv = 0.f;
      if (d < dk) {
        const long row = row0 + t0 + tt;
        kv = ldf(k + row * k_stride + hd * dk + d);
        qv = ldf(q + row * q_stride + hd * dk + d);
        if (silu) { kv = silu_f(kv); qv = silu_f(qv); }
        qv *= q_scale;
      }
      sk[tt][d] = kv;
      sq[tt][d] = qv;
    }
    for (int idx = tid; idx < nt * 64; idx += 256) {
      const int tt = idx >> 6, jj = idx & 63;
      float vv = 0.f;
      if (c0 + jj < dv) {
        vv = ldf(v + static_cast<long>(row0 + t0 + tt) * v_stride + hd * dv + c0 + jj);
        if (silu) vv = silu_f(vv);
      }
      sv[tt][jj] = vv;
    }
    if (MLSTM && tid == 0) {
      for (int tt = 0; tt < nt; ++tt) {
        const float* gp = gates + static_cast<long>(row0 + t0 + tt) * (2 * H);
        const float ig = gate_cap * tanhf(gp[hd] / gate_cap);
        const float fg = logsigmoid_f(gate_cap * tanhf(gp[H + hd] / gate_cap));
        const float m_new = fmaxf(fg + m, ig);
        fsum += fg;
        sfa[tt] = expf(fg + m - m_new);  // pass 1, first token: m = -inf gives 0
        sia[tt] = expf(ig - m_new);
        sem[tt] = expf(-m_new);
        m = m_new;
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = sv[tt][j];
      float part = 0.f, pn = 0.f;
      if (MLSTM) {
        const float fa = sfa[tt], ia = sia[tt];
        const float vi = ia * vj;
#pragma unroll
        for (int i = 0; i < DR; ++i) {
          const float kd = sk[tt][r * DR + i], qd = sq[tt][r * DR + i];
          S[i] = fa * S[i] + kd * vi;
          nvec[i] = fa * nvec[i] + ia * kd;
          part += S[i] * qd;
          pn += nvec[i] * qd;
        }
        if (j == 0) redn[tt][r] = pn;
      } else {
#pragma unroll
        for (int i = 0; i < DR; ++i) {
          const float kd = sk[tt][r * DR + i], qd = sq[tt][r * DR + i];
          S[i] = a * S[i] + kd * vj;
          part += S[i] * qd;
        }
      }
      red[tt][r][j] = part;
    }
    if (mode == 1) continue;  // pass 1 keeps the end state only (uniform: the next stage starts with a barrier)
    __syncthreads();
    for (int idx = tid; idx < nt * 64; idx += 256) {
      const int tt = idx >> 6, jj = idx & 63;
      if (c0 + jj >= dv) continue;
      float o = (red[tt][0][jj] + red[tt][1][jj]) + (red[tt][2][jj] + red[tt][3][jj]);
      if (MLSTM) {
        const float nq = (redn[tt][0] + redn[tt][1]) + (redn[tt][2] + redn[tt][3]);
        o = o / (fmaxf(fabsf(nq), sem[tt]) + 1e-6f);
      }
      out[static_cast<long>(row0 + t0 + tt) * HV + hd * dv + c0 + jj] = o;
    }
  }
  if (!write_state) return;
#pragma unroll
  for (int i = 0; i < DR; ++i) {
    const int d = r * DR + i;
    if (d < dk && col_ok) dst[oS + static_cast<long>(d) * dv + col] = S[i];
    if (MLSTM && blockIdx.z == 0 && j == 0 && d < dk) dst[oN + d] = nvec[i];
  }
  if (MLSTM && blockIdx.z == 0 && tid == 0) {
    dst[oM] = m;
    if (mode == 1) dst[oM + H] = fsum;  // [H] sums after the [H] maxima
  }
}

// Chains the pieces: sc_start[s][p] = the state at the start of piece p, from the slot (or zero for a
// sequence's first tokens) and the end states sc_local[s][0..p-1] of pass 1.  One thread per state
// element (S, then n; the head's scalars are recomputed by every thread); pieces walked in order.
template <bool MLSTM>
__global__ void __launch_bounds__(256) scan_chain_kernel(const float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ state_rows, long off,
                                                         const int* __restrict__ qsl, const int* __restrict__ seq_lens,
                                                         const float* __restrict__ decay, int n_rows, int H, int dk,
                                                         int dv, int piece, int npieces, const float* __restrict__ sc_local,
                                                         float* __restrict__ sc_start, long sc_floats) {
  const int s = blockIdx.x, hd = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;  // element of the head: S [dk*dv], then n [dk]
  const int nS = dk * dv, nE = nS + (MLSTM ? dk : 0);
  if (e >= nE) return;
  const int row0 = qsl[s];
  if (row0 < 0 || row0 >= n_rows) return;
  const int qlen = min(qsl[s + 1], n_rows) - row0;
  if (qlen <= 0) return;
  const int np = min((qlen + piece - 1) / piece, npieces);
  const bool fresh = seq_lens[s] - qlen == 0;
  const long oE = e < nS ? static_cast<long>(hd) * nS + e : static_cast<long>(H) * nS + static_cast<long>(hd) * dk + (e - nS);
  const long oM = static_cast<long>(H) * nS + static_cast<long>(H) * dk + hd;
  const float* slot = state + static_cast<long>(state_rows[s]) * state_stride + off;
  float cur = fresh ? 0.f : slot[oE];
  float m = (MLSTM && !fresh) ? slot[oM] : 0.f;
  const float ap = MLSTM ? 0.f : powf(decay[hd], static_cast<float>(piece));
  for (int p = 0; p < np; ++p) {
    const long at = (static_cast<long>(s) * npieces + p) * sc_floats;
    sc_start[at + oE] = cur;
    if (MLSTM && e == 0) sc_start[at + oM] = m;
    if (p == np - 1) break;
    const float loc = sc_local[at + oE];
    if (MLSTM) {
      const float m_loc = sc_local[at + oM], fs = sc_local[at + oM + H];
      const float m_new = fmaxf(fs + m, m_loc);
      cur = expf(fs + m - m_new) * cur + expf(m_loc - m_new) * loc;
      m = m_new;
    } else {
      cur = ap * cur + loc;
    }
  }
}

template <typename T, bool MLSTM>
static bool launch_scan_t(float* out, const T* q, long qs, const T* k, long ks, const T* v, long vs, const float* decay,
                          const float* gates, float* state, long state_stride, const int* state_rows, long off,
                          const int* qsl, const int* seq_lens, int S, int n_rows, int H, int dk, int dv, int silu, float cap,
                          float q_scale, int piece, int npieces, int mode, float* sc_local, float* sc_start,
                          long sc_floats, hipStream_t st) {
  const dim3 grid(S * npieces, H, (dv + 63) / 64), block(256);
#define MIX_SCAN(DR)                                                                                               \
  hipLaunchKernelGGL((matrix_scan_kernel<T, DR, MLSTM>), grid, block, 0, st, out, q, qs, k, ks, v, vs, decay, gates, \
                     state, state_stride, state_rows, off, qsl, seq_lens, n_rows, H, dk, dv, silu, cap, q_scale, piece, npieces, \
                     mode, sc_local, sc_start, sc_floats)
  if (dk <= 32) MIX_SCAN(8);
  else if (dk <= 64) MIX_SCAN(16);
  else if (dk <= 128) MIX_SCAN(32);
  else if (dk <= 256) MIX_SCAN(64);
  else return false;
#undef MIX_SCAN
  MXS_CHECK_LAUNCH();
  return true;
}

bool launch_matrix_scan_pass(float*, const void*, long, const void*, long, const void*, long, const float*, const float*,
                             float*, long, const int*, long, const int*, const int*, int, int, int, int, int, int, float,
                             float, bool, bool, int, int, int, float*, float*, long, hipStream_t);

bool launch_matrix_scan(float* out, const void* q, long qs, const void* k, long ks, const void* v, long vs,
                        const float* decay, const float* gates, float* state, long state_stride, const int* state_rows,
                        long off, const int* qsl, const int* seq_lens, int S, int n_rows, int H, int dk, int dv, int silu,
                        float cap, float q_scale, bool mlstm, bool bf, int piece, int npieces, float* sc_local,
                        float* sc_start, long sc_floats, hipStream_t st) {
  if (S == 0) return true;
  if (dk > 256) return false;
  if (npieces > 1) {  // pass 1, chain, pass 2
    if (!launch_matrix_scan_pass(out, q, qs, k, ks, v, vs, decay, gates, state, state_stride, state_rows, off, qsl,
                                 seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, mlstm, bf, piece, npieces, 1,
                                 sc_local, sc_start, sc_floats, st))
      return false;
    const dim3 grid(S, H, (dk * dv + (mlstm ? dk : 0) + 255) / 256);
    if (mlstm)
      hipLaunchKernelGGL(scan_chain_kernel<true>, grid, dim3(256), 0, st, state, state_stride, state_rows, off, qsl,
                         seq_lens, decay, n_rows, H, dk, dv, piece, npieces, sc_local, sc_start, sc_floats);
    else
      hipLaunchKernelGGL(scan_chain_kernel<false>, grid, dim3(256), 0, st, state, state_stride, state_rows, off, qsl,
                         seq_lens, decay, n_rows, H, dk, dv, piece, npieces, sc_local, sc_start, sc_floats);
    MXS_CHECK_LAUNCH();
    return launch_matrix_scan_pass(out, q, qs, k, ks, v, vs, decay, gates, state, state_stride, state_rows, off, qsl,
                                   seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, mlstm, bf, piece, npieces, 2,
                                   sc_local, sc_start, sc_floats, st);
  }
  return launch_matrix_scan_pass(out, q, qs, k, ks, v, vs, decay, gates, state, state_stride, state_rows, off, qsl,
                                 seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, mlstm, bf, 1, 1, 0, nullptr, nullptr,
                                 0, st);
}

bool launch_matrix_scan_pass(float* out, const void* q, long qs, const void* k, long ks, const void* v, long vs,
                             const float* decay, const float* gates, float* state, long state_stride,
                             const int* state_rows, long off, const int* qsl, const int* seq_lens, int S, int n_rows,
                             int H, int dk, int dv, int silu, float cap, float q_scale, bool mlstm, bool bf, int piece,
                             int npieces, int mode, float* sc_local, float* sc_start, long sc_floats, hipStream_t st) {
  if (bf) {
    using T = bf16_t;
    return mlstm ? launch_scan_t<T, true>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                          state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, piece, npieces, mode,
                                          sc_local, sc_start, sc_floats, st)
                 : launch_scan_t<T, false>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                           state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, piece, npieces, mode,
                                          sc_local, sc_start, sc_floats, st);
  }
  using T = float;
  return mlstm ? launch_scan_t<T, true>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                        state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, piece, npieces, mode,
                                          sc_local, sc_start, sc_floats, st)
               : launch_scan_t<T, false>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                         state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, piece, npieces, mode,
                                          sc_local, sc_start, sc_floats, st);
}

}  // namespace mxs
