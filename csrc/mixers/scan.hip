// Token-by-token recurrences with a matrix state per head (gfx950): decayed linear attention and
// the mLSTM memory.  The state S [dk, dv] of one (sequence, head) is split over workgroups by
// 64-column slices (columns never interact) and inside a workgroup over 4 waves by rows: thread
// (r, j) keeps rows r*DR .. r*DR+DR-1 of column j in registers for the whole chunk, so a step is
// DR fused multiply-adds for the update, DR for the read-out, and one 4-way sum through LDS.
// Tokens are staged 16 at a time (q, k rows and the v slice as fp32 in LDS, activations applied),
// two barriers per 16 tokens.  The sum order of a token's output does not depend on where a chunk
// starts or ends, so cutting a prompt differently gives the same bits.
// State, decays, gates and every product are fp32; q, k, v come as bf16 or fp32.
#include "mix_common.h"

namespace mxs {

constexpr int kTB = 16;  // tokens per LDS stage

template <typename T, int DR, bool MLSTM>
__global__ void __launch_bounds__(256) matrix_scan_kernel(
    float* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride, const float* __restrict__ decay, const float* __restrict__ gates,
    float* __restrict__ state, long state_stride, const int* __restrict__ state_rows, long off,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, int n_rows, int H, int dk, int dv, int silu,
    float gate_cap, float q_scale) {
  constexpr int DT = 4 * DR;  // padded key size
  __shared__ float sk[kTB][DT];
  __shared__ float sq[kTB][DT];
  __shared__ float sv[kTB][64];
  __shared__ float red[kTB][4][64];
  __shared__ float redn[kTB][4];
  __shared__ float sfa[kTB], sia[kTB], sem[kTB];
  const int s = blockIdx.x, hd = blockIdx.y, c0 = blockIdx.z * 64;
  const int tid = threadIdx.x, j = tid & 63, r = tid >> 6;
  const int row0 = qsl[s];
  if (row0 < 0 || row0 >= n_rows) return;
  const int qlen = min(qsl[s + 1], n_rows) - row0;  // never past the step's rows, whatever the metadata says
  if (qlen <= 0) return;
  const bool fresh = seq_lens[s] - qlen == 0;  // the sequence's first tokens: zero state
  const int col = c0 + j;
  const bool col_ok = col < dv;
  float* sbase = state + static_cast<long>(state_rows[s]) * state_stride + off;
  float* Sg = sbase + static_cast<long>(hd) * dk * dv;
  float* ng = sbase + static_cast<long>(H) * dk * dv + static_cast<long>(hd) * dk;
  float* mg = sbase + static_cast<long>(H) * dk * dv + static_cast<long>(H) * dk + hd;
  float S[DR], nvec[DR];
#pragma unroll
  for (int i = 0; i < DR; ++i) {
    const int d = r * DR + i;
    S[i] = (!fresh && d < dk && col_ok) ? Sg[static_cast<long>(d) * dv + col] : 0.f;
    nvec[i] = (MLSTM && !fresh && d < dk) ? ng[d] : 0.f;
  }
  float m = (MLSTM && !fresh) ? *mg : 0.f;  // used by thread 0 only
  const float a = MLSTM ? 0.f : decay[hd];
  const int HV = H * dv;
  for (int t0 = 0; t0 < qlen; t0 += kTB) {
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
        sfa[tt] = expf(fg + m - m_new);
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
#pragma unroll
  for (int i = 0; i < DR; ++i) {
    const int d = r * DR + i;
    if (d < dk && col_ok) Sg[static_cast<long>(d) * dv + col] = S[i];
    if (MLSTM && blockIdx.z == 0 && j == 0 && d < dk) ng[d] = nvec[i];
  }
  if (MLSTM && blockIdx.z == 0 && tid == 0) *mg = m;
}

template <typename T, bool MLSTM>
static bool launch_scan_t(float* out, const T* q, long qs, const T* k, long ks, const T* v, long vs, const float* decay,
                          const float* gates, float* state, long state_stride, const int* state_rows, long off,
                          const int* qsl, const int* seq_lens, int S, int n_rows, int H, int dk, int dv, int silu, float cap,
                          float q_scale, hipStream_t st) {
  const dim3 grid(S, H, (dv + 63) / 64), block(256);
#define MIX_SCAN(DR)                                                                                               \
  hipLaunchKernelGGL((matrix_scan_kernel<T, DR, MLSTM>), grid, block, 0, st, out, q, qs, k, ks, v, vs, decay, gates, \
                     state, state_stride, state_rows, off, qsl, seq_lens, n_rows, H, dk, dv, silu, cap, q_scale)
  if (dk <= 32) MIX_SCAN(8);
  else if (dk <= 64) MIX_SCAN(16);
  else if (dk <= 128) MIX_SCAN(32);
  else if (dk <= 256) MIX_SCAN(64);
  else return false;
#undef MIX_SCAN
  MXS_CHECK_LAUNCH();
  return true;
}

bool launch_matrix_scan(float* out, const void* q, long qs, const void* k, long ks, const void* v, long vs,
                        const float* decay, const float* gates, float* state, long state_stride, const int* state_rows,
                        long off, const int* qsl, const int* seq_lens, int S, int n_rows, int H, int dk, int dv, int silu,
                        float cap, float q_scale, bool mlstm, bool bf, hipStream_t st) {
  if (S == 0) return true;
  if (bf) {
    using T = bf16_t;
    return mlstm ? launch_scan_t<T, true>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                          state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, st)
                 : launch_scan_t<T, false>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                           state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, st);
  }
  using T = float;
  return mlstm ? launch_scan_t<T, true>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                        state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, st)
               : launch_scan_t<T, false>(out, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, decay, gates, state,
                                         state_stride, state_rows, off, qsl, seq_lens, S, n_rows, H, dk, dv, silu, cap, q_scale, st);
}

}  // namespace mxs
