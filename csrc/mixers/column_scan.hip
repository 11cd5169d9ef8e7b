// Token-by-token recurrences whose state columns never interact (gfx950): the selective state space
// with a scalar decay per head and token, and the gated delta rule with a decay per key channel.
//
// The state S [dk, dv] of one (sequence, head) is stored transposed, [dv][dk], and split over
// workgroups by 16 columns.  A column belongs to 16 neighbouring lanes (one DPP row); each keeps R
// consecutive rows of it in registers for the whole chunk, so the delta rule's S^T k, which needs a
// column's full sum BEFORE the update, is R multiply-adds and four DPP row rotations, with no LDS
// round trip or barrier inside a token.  Sixteen tokens are staged per barrier pair: the key-side
// vectors as fp32 in LDS with everything that is per token and head already applied (unit norm,
// query scale, decays through softplus and exp, write strength), the 16 value columns, and the
// previous 16 tokens' outputs are written while the next are staged.
// A token's sums run in an order fixed by the sizes alone, so cutting a prompt differently gives the
// same bits.  State, decays, gates and every product are fp32; the operands come as bf16 or fp32.
#include "mix_common.h"
#include "column_scan.h"

namespace mxs {

constexpr int kST = 16;    // tokens per LDS stage
constexpr int kCols = 16;  // state columns per workgroup (4 per wave, 16 lanes each)

__device__ __forceinline__ float softplus_cs(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// sum over the 16 lanes of a DPP row, the same bits in every lane (row rotations by 8, 4, 2, 1)
__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
  return v;
}

template <typename T, int R, bool DELTA>
__global__ void __launch_bounds__(256) column_scan_kernel(const ScanArgs p) {
  constexpr int DK = 16 * R;  // padded key size
  __shared__ float sk[kST][DK];
  __shared__ float sq[kST][DK];
  __shared__ float sg[DELTA ? kST : 1][DELTA ? DK : 1];
  __shared__ float sv[kST][kCols];
  __shared__ float so[kST][kCols];
  __shared__ float sb[kST], sa[kST];
  const int s = blockIdx.x, hd = blockIdx.y, c0 = blockIdx.z * kCols;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int rp = lane & 15, cl = wid * 4 + (lane >> 4);  // row part; column inside the workgroup
  const int H = p.H, dk = p.dk, dv = p.dv;
  const int row0 = p.qsl[s];
  if (row0 < 0 || row0 >= p.n_rows) return;
  const int qlen = min(p.qsl[s + 1], p.n_rows) - row0;  // never past the step's rows, whatever the metadata says
  if (qlen <= 0) return;
  const bool fresh = p.seq_lens[s] - qlen <= 0;
  const int col = c0 + cl;
  const bool col_ok = col < dv;
  const int kh = hd / (H / p.G);  // the head's q/k head (delta) or B/C group (ssd)
  float* Sg = p.state + static_cast<long>(p.state_rows[s]) * p.state_stride + p.off +
              (static_cast<long>(hd) * dv + (col_ok ? col : 0)) * dk + rp * R;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (!fresh && col_ok && rp * R + i < dk) ? Sg[i] : 0.f;
  const T* qp = static_cast<const T*>(p.q);
  const T* kp = static_cast<const T*>(p.k);
  const T* vp = static_cast<const T*>(p.v);
  const T* bp = static_cast<const T*>(p.beta);
  const T* ap = static_cast<const T*>(p.a);
  const float eA = expf(p.A_log[hd]);
  const float Dh = DELTA ? 0.f : p.D[hd];
  const int HV = H * dv;
  int prev_t0 = -1, prev_nt = 0;
  for (int t0 = 0; t0 < qlen; t0 += kST) {
    const int nt = min(kST, qlen - t0);
    __syncthreads();  // the previous stage's reads of the staged vectors and writes of so are done
    if (prev_t0 >= 0) {
      const int tt = tid >> 4, jj = tid & 15;
      if (tt < prev_nt && c0 + jj < dv) p.out[static_cast<long>(row0 + prev_t0 + tt) * HV + hd * dv + c0 + jj] = so[tt][jj];
    }
    // key-side vectors: wave w stages tokens w, w+4, ...
    for (int tt = wid; tt < nt; tt += 4) {
      const long row = row0 + t0 + tt;
      if (DELTA) {
        float kq[2][(DK + 63) / 64];
        float ssk = 0.f, ssq = 0.f;
#pragma unroll
        for (int c = 0; c < (DK + 63) / 64; ++c) {
          const int d = lane + 64 * c;
          const float kv = d < dk ? ldf(kp + row * p.k_stride + kh * dk + d) : 0.f;
          const float qv = d < dk ? ldf(qp + row * p.q_stride + kh * dk + d) : 0.f;
          kq[0][c] = kv;
          kq[1][c] = qv;
          ssk += kv * kv;
          ssq += qv * qv;
        }
        const float ik = rsqrtf(wave_sum(ssk) + p.unit_eps), iq = rsqrtf(wave_sum(ssq) + p.unit_eps) * p.q_scale;
#pragma unroll
        for (int c = 0; c < (DK + 63) / 64; ++c) {
          const int d = lane + 64 * c;
          if (d < DK) {
            sk[tt][d] = kq[0][c] * ik;
            sq[tt][d] = kq[1][c] * iq;
            sg[tt][d] = d < dk ? expf(-eA * softplus_cs(ldf(ap + row * p.a_stride + hd * dk + d) + p.dt_bias[hd * dk + d])) : 0.f;
          }
        }
        if (lane == 0) sb[tt] = sigmoid_f(ldf(bp + row * p.beta_stride + hd));
      } else {
        for (int d = lane; d < DK; d += 64) {
          sk[tt][d] = d < dk ? ldf(kp + row * p.k_stride + kh * dk + d) : 0.f;
          sq[tt][d] = d < dk ? ldf(qp + row * p.q_stride + kh * dk + d) : 0.f;
        }
        if (lane == 0) {
          const float dt = softplus_cs(ldf(bp + row * p.beta_stride + hd) + p.dt_bias[hd]);
          sb[tt] = dt;
          sa[tt] = expf(-eA * dt);
        }
      }
    }
    {
      const int tt = tid >> 4, jj = tid & 15;
      sv[tt][jj] = (tt < nt && c0 + jj < dv) ? ldf(vp + static_cast<long>(row0 + t0 + tt) * p.v_stride + hd * dv + c0 + jj) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = sv[tt][cl];
      const float* kr = &sk[tt][rp * R];
      const float* qr = &sq[tt][rp * R];
      float o;
      if (DELTA) {
        const float* gr = &sg[tt][rp * R];
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
          S[i] *= gr[i];
          part += S[i] * kr[i];
        }
        const float u = sb[tt] * (vj - row16_sum(part));
        part = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
          S[i] += kr[i] * u;
          part += S[i] * qr[i];
        }
        o = row16_sum(part);
      } else {
        const float a = sa[tt], xb = sb[tt] * vj;
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
          S[i] = a * S[i] + xb * kr[i];
          part += S[i] * qr[i];
        }
        o = row16_sum(part) + Dh * vj;
      }
      if (rp == 0) so[tt][cl] = o;
    }
    prev_t0 = t0;
    prev_nt = nt;
  }
  __syncthreads();
  {
    const int tt = tid >> 4, jj = tid & 15;
    if (tt < prev_nt && c0 + jj < dv) p.out[static_cast<long>(row0 + prev_t0 + tt) * HV + hd * dv + c0 + jj] = so[tt][jj];
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (rp * R + i < dk) Sg[i] = S[i];
  }
}

template <typename T, bool DELTA>
static bool launch_cs(const ScanArgs& a, int S, hipStream_t st) {
  const dim3 grid(S, a.H, (a.dv + kCols - 1) / kCols), block(256);
#define MIX_CS(R) hipLaunchKernelGGL((column_scan_kernel<T, R, DELTA>), grid, block, 0, st, a)
  if (a.dk <= 32) MIX_CS(2);
  else if (a.dk <= 64) MIX_CS(4);
  else if (a.dk <= 128) MIX_CS(8);
  else if (a.dk <= 256) MIX_CS(16);
  else return false;
#undef MIX_CS
  MXS_CHECK_LAUNCH();
  return true;
}

bool launch_column_scan(const ScanArgs& a, int S, bool delta, bool bf, hipStream_t st) {
  if (S == 0 || a.n_rows == 0) return true;
  if (bf) return delta ? launch_cs<bf16_t, true>(a, S, st) : launch_cs<bf16_t, false>(a, S, st);
  return delta ? launch_cs<float, true>(a, S, st) : launch_cs<float, false>(a, S, st);
}

}  // namespace mxs
