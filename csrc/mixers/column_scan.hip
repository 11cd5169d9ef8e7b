// Token-by-token recurrences whose state columns never interact (gfx950): the selective state space
// with a scalar decay per head and token, and the gated delta rule with a decay per key channel.
//
// The state S [dk, dv] of one (sequence, head) is stored transposed, [dv][dk], and split over
// workgroups by 16 columns.  A column belongs to 16 neighbouring lanes (one DPP row); each keeps R
// consecutive rows of it in registers for the whole chunk, so the delta rule's S^T k, which needs a
// column's full sum BEFORE the update, is R multiply-adds and four DPP row rotations, with no LDS
// round trip or barrier inside a token.  Sixteen tokens are staged per barrier pair: the key-side
// vectors as fp32 in LDS with everything that is per token and head already applied (unit norm,
// query scale, decays through softplus and exp, write strength) and the 16 value columns.  The 256
// threads stage as 16 tokens x 16 runs, the same 16-lane rows as the recurrence, so a unit norm is
// a DPP row sum too; a stage's global loads are issued before the stage before it is walked, and
// the previous 16 tokens' outputs are written while the next are staged.
// Long chunks are cut into pieces that run side by side: pass 1 runs every piece from an empty state
// and keeps its end state, and what carries a state across the piece (state space: the summed decay
// exponents; delta rule: the piece's dk x dk transition matrix, from dk more columns started as the
// identity); the states at the pieces' starts are chained from those; pass 2 runs every piece again
// from its true start and writes the outputs.
// A token's sums run in an order fixed by the sizes alone, so cutting a prompt differently gives the
// same bits.  State, decays, gates and every product are fp32; the operands come as bf16 or fp32.
#include <algorithm>

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

// R consecutive elements as fp32; `vec`: the run is aligned to its own size (16 bytes at most)
template <int R> __device__ __forceinline__ void load_run(const bf16_t* p, float* o, bool vec) {
  if (vec) {
    if constexpr (R >= 8) {
#pragma unroll
      for (int c = 0; c < R / 8; ++c) {
        const uint4 a = *reinterpret_cast<const uint4*>(p + 8 * c);
        o[8 * c] = bf2f_lo(a.x); o[8 * c + 1] = bf2f_hi(a.x); o[8 * c + 2] = bf2f_lo(a.y); o[8 * c + 3] = bf2f_hi(a.y);
        o[8 * c + 4] = bf2f_lo(a.z); o[8 * c + 5] = bf2f_hi(a.z); o[8 * c + 6] = bf2f_lo(a.w); o[8 * c + 7] = bf2f_hi(a.w);
      }
    } else if constexpr (R == 4) {
      const uint2 a = *reinterpret_cast<const uint2*>(p);
      o[0] = bf2f_lo(a.x); o[1] = bf2f_hi(a.x); o[2] = bf2f_lo(a.y); o[3] = bf2f_hi(a.y);
    } else {
      const uint32_t a = *reinterpret_cast<const uint32_t*>(p);
      o[0] = bf2f_lo(a); o[1] = bf2f_hi(a);
    }
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) o[i] = bf2f(p[i]);
  }
}
template <int R> __device__ __forceinline__ void load_run(const float* p, float* o, bool vec) {
  if (vec) {
    if constexpr (R >= 4) {
#pragma unroll
      for (int c = 0; c < R / 4; ++c) {
        const float4 a = *reinterpret_cast<const float4*>(p + 4 * c);
        o[4 * c] = a.x; o[4 * c + 1] = a.y; o[4 * c + 2] = a.z; o[4 * c + 3] = a.w;
      }
    } else {
      const float2 a = *reinterpret_cast<const float2*>(p);
      o[0] = a.x; o[1] = a.y;
    }
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) o[i] = p[i];
  }
}
template <int R> __device__ __forceinline__ void store_run(float* p, const float* o, bool vec) {
  if (vec) {
    if constexpr (R >= 4) {
#pragma unroll
      for (int c = 0; c < R / 4; ++c) *reinterpret_cast<float4*>(p + 4 * c) = make_float4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
    } else {
      *reinterpret_cast<float2*>(p) = make_float2(o[0], o[1]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) p[i] = o[i];
  }
}

// What one thread brings in for a stage: its run of R key-side elements of the token it stages (the
// token tid / 16; the run is the one whose rows it owns in the recurrence), one value element and the
// token's scalar.  The loads of a stage are issued before the 16 tokens of the stage before it are
// walked, so their latency hides behind that walk.
template <int R, bool DELTA, int CG> struct StageRegs {
  float k[R], q[R], a[DELTA ? R : 1], v[CG], b;
};

template <typename T, int R, bool DELTA, int CG>
__device__ __forceinline__ void load_stage(StageRegs<R, DELTA, CG>& r, const ScanArgs& p, long row, bool ok, int kh, int hd,
                                           int rp, int vcol, int flags) {
  const T* qp = static_cast<const T*>(p.q);
  const T* kp = static_cast<const T*>(p.k);
  const T* vp = static_cast<const T*>(p.v);
  const T* bp = static_cast<const T*>(p.beta);
  const T* ap = static_cast<const T*>(p.a);
  const int d0 = rp * R;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    r.k[i] = 0.f;
    r.q[i] = 0.f;
    if (DELTA) r.a[i] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < CG; ++j) r.v[j] = 0.f;
  r.b = 0.f;
  if (!ok) return;
  if (d0 + R <= p.dk) {
    load_run<R>(kp + row * p.k_stride + kh * p.dk + d0, r.k, flags & 1);
    load_run<R>(qp + row * p.q_stride + kh * p.dk + d0, r.q, flags & 2);
    if (DELTA) load_run<R>(ap + row * p.a_stride + hd * p.dk + d0, r.a, flags & 4);
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (d0 + i < p.dk) {
        r.k[i] = ldf(kp + row * p.k_stride + kh * p.dk + d0 + i);
        r.q[i] = ldf(qp + row * p.q_stride + kh * p.dk + d0 + i);
        if (DELTA) r.a[i] = ldf(ap + row * p.a_stride + hd * p.dk + d0 + i);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < CG; ++j)
    if (vcol + j * kCols < p.dv) r.v[j] = ldf(vp + row * p.v_stride + hd * p.dv + vcol + j * kCols);
  r.b = ldf(bp + row * p.beta_stride + hd);
}

// ST: tokens per stage, 16, or 1 for steps of single tokens only.  CG: groups of 16 columns a workgroup
// takes, each thread one column of every group: a step of single tokens is a read and a write of the
// state and little else, so its workgroups take 64 columns and have four times the bytes in flight.
template <typename T, int R, bool DELTA, int ST, int CG>
__global__ void __launch_bounds__(256) column_scan_kernel(const ScanArgs p, int flags) {
  constexpr int DK = 16 * R;  // padded key size
  __shared__ __attribute__((aligned(16))) float sk[ST][DK];
  __shared__ __attribute__((aligned(16))) float sq[ST][DK];
  __shared__ __attribute__((aligned(16))) float sg[DELTA ? ST : 1][DELTA ? DK : 4];
  constexpr int WC = kCols * CG;  // columns per workgroup
  __shared__ float sv[ST][WC];
  __shared__ float so[ST][WC];
  __shared__ float sb[ST], sa[kST];
  const int mode = p.mode, np = p.npieces;
  // neighbouring workgroups take neighbouring columns of one head's state: consecutive memory
  const int s = blockIdx.z / np, pc = blockIdx.z - s * np, hd = blockIdx.y, c0 = blockIdx.x * WC;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  // recurrence: the thread owns rows rp*R.. of column cl.  staging: run rp of token cl.
  const int rp = lane & 15, cl = wid * 4 + (lane >> 4);
  const int H = p.H, dk = p.dk, dv = p.dv;
  int row0 = p.qsl[s];
  if (row0 < 0 || row0 >= p.n_rows) return;
  const int qlen_all = min(p.qsl[s + 1], p.n_rows) - row0;  // never past the step's rows, whatever the metadata says
  const int tb = mode == 0 ? 0 : pc * p.piece;              // this workgroup's rows of the chunk: [tb, te)
  const int te = mode == 0 ? qlen_all : min(qlen_all, tb + p.piece);
  if (te <= tb) return;
  const int qlen = te - tb;
  row0 += tb;
  const bool fresh = mode == 1 || (mode == 0 && p.seq_lens[s] - qlen_all <= 0);
  // delta rule, pass 1: dk more columns, started as the identity and fed no values, end as the piece's
  // transition matrix (the state at the piece's end is that matrix times the state at its start, plus
  // the end state from an empty start)
  const int ncols = (DELTA && mode == 1) ? dv + dk : dv;
  const int kh = hd / (H / p.G);  // the head's q/k head (delta rule) or B/C group (state space)
  const long sc_at = (static_cast<long>(s) * np + pc) * (static_cast<long>(H) * dv * dk);
  float* slot = p.state + static_cast<long>(p.state_rows[s]) * p.state_stride + p.off;
  const float* Sin0 = mode == 2 ? p.sc_start + sc_at : slot;
  float* Sout0 = mode == 1 ? p.sc_local + (static_cast<long>(s) * np + pc) * (static_cast<long>(H) * ncols * dk) : slot;
  const int out_cols = mode == 1 ? ncols : dv;  // columns per head where the state goes
  const bool write_state = mode != 2 || te == qlen_all;
  const bool run_in = rp * R + R <= dk;
  float S[CG][R];
#pragma unroll
  for (int j = 0; j < CG; ++j) {  // every group's loads are issued before any is waited for
    const int col = c0 + j * kCols + cl;
#pragma unroll
    for (int i = 0; i < R; ++i) S[j][i] = 0.f;
    if (!fresh && col < dv) {
      const float* Sin = Sin0 + (static_cast<long>(hd) * dv + col) * dk + rp * R;
      if (run_in) {
        load_run<R>(Sin, S[j], flags & 8);
      } else {
#pragma unroll
        for (int i = 0; i < R; ++i)
          if (rp * R + i < dk) S[j][i] = Sin[i];
      }
    }
    if (DELTA && mode == 1 && col >= dv) {
#pragma unroll
      for (int i = 0; i < R; ++i) S[j][i] = rp * R + i == col - dv ? 1.f : 0.f;
    }
  }
  float dsum = 0.f;  // state space, mode 1: this thread's share of the piece's summed decay exponents
  const float eA = expf(p.A_log[hd]);
  const float Dh = DELTA ? 0.f : p.D[hd];
  float bias[DELTA ? R : 1];
  if (DELTA) {
#pragma unroll
    for (int i = 0; i < R; ++i) bias[i] = rp * R + i < dk ? p.dt_bias[hd * dk + rp * R + i] : 0.f;
  } else {
    bias[0] = p.dt_bias[hd];
  }
  const int HV = H * dv;
  StageRegs<R, DELTA, CG> rg;
  load_stage<T, R, DELTA, CG>(rg, p, row0 + cl, cl < ST && cl < qlen, kh, hd, rp, c0 + rp, flags);
  int prev_t0 = -1, prev_nt = 0;
  for (int t0 = 0; t0 < qlen; t0 += ST) {
    const int nt = min(ST, qlen - t0);
    __syncthreads();  // the previous stage's reads of the staged vectors and writes of so are done
    if (mode != 1 && prev_t0 >= 0 && cl < prev_nt) {
#pragma unroll
      for (int j = 0; j < CG; ++j)
        if (c0 + j * kCols + rp < dv)
          p.out[static_cast<long>(row0 + prev_t0 + cl) * HV + hd * dv + c0 + j * kCols + rp] = so[cl][j * kCols + rp];
    }
    // this stage's registers -> LDS, with everything that is per token and head applied
    if (cl >= ST) {
      // ST = 1: the other fifteen token rows of the staging layout have nothing to bring
    } else if (DELTA) {
      float ssk = 0.f, ssq = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        ssk += rg.k[i] * rg.k[i];
        ssq += rg.q[i] * rg.q[i];
      }
      const float ik = rsqrtf(row16_sum(ssk) + p.unit_eps), iq = rsqrtf(row16_sum(ssq) + p.unit_eps) * p.q_scale;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        sk[cl][rp * R + i] = rg.k[i] * ik;
        sq[cl][rp * R + i] = rg.q[i] * iq;
        sg[cl][rp * R + i] = rp * R + i < dk ? expf(-eA * softplus_cs(rg.a[i] + bias[i])) : 0.f;
      }
      if (rp == 0) sb[cl] = sigmoid_f(rg.b);
    } else {
#pragma unroll
      for (int i = 0; i < R; ++i) {
        sk[cl][rp * R + i] = rg.k[i];
        sq[cl][rp * R + i] = rg.q[i];
      }
      if (rp == 0) {
        const float dt = softplus_cs(rg.b + bias[0]);
        sb[cl] = dt;
        sa[cl] = expf(-eA * dt);
        if (cl < nt) dsum += eA * dt;
      }
    }
    if (cl < ST) {
#pragma unroll
      for (int j = 0; j < CG; ++j) sv[cl][j * kCols + rp] = rg.v[j];
    }
    __syncthreads();
    if (t0 + ST < qlen)  // the next stage's loads fly while this stage's tokens are walked
      load_stage<T, R, DELTA, CG>(rg, p, row0 + t0 + ST + cl, cl < ST && t0 + ST + cl < qlen, kh, hd, rp, c0 + rp, flags);
    const bool readout = mode != 1;  // pass 1 wants a piece's end state only
    auto token = [&](int tt) {
      const float* kr = &sk[tt][rp * R];
      const float* qr = &sq[tt][rp * R];
#pragma unroll
      for (int j = 0; j < CG; ++j) {
      float* Sj = S[j];
      const float vj = sv[tt][j * kCols + cl];
      float o;
      if (DELTA) {
        const float* gr = &sg[tt][rp * R];
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int i = 0; i < R; i += 2) {
          Sj[i] *= gr[i];
          Sj[i + 1] *= gr[i + 1];
          p0 += Sj[i] * kr[i];
          p1 += Sj[i + 1] * kr[i + 1];
        }
        const float u = sb[tt] * (vj - row16_sum(p0 + p1));
        if (readout) {
          p0 = 0.f;
          p1 = 0.f;
#pragma unroll
          for (int i = 0; i < R; i += 2) {
            Sj[i] += kr[i] * u;
            Sj[i + 1] += kr[i + 1] * u;
            p0 += Sj[i] * qr[i];
            p1 += Sj[i + 1] * qr[i + 1];
          }
          o = row16_sum(p0 + p1);
        } else {
#pragma unroll
          for (int i = 0; i < R; ++i) Sj[i] += kr[i] * u;
          o = 0.f;
        }
      } else if (readout) {
        const float a = sa[tt], xb = sb[tt] * vj;
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int i = 0; i < R; i += 2) {
          Sj[i] = a * Sj[i] + xb * kr[i];
          Sj[i + 1] = a * Sj[i + 1] + xb * kr[i + 1];
          p0 += Sj[i] * qr[i];
          p1 += Sj[i + 1] * qr[i + 1];
        }
        o = row16_sum(p0 + p1) + Dh * vj;
      } else {
        const float a = sa[tt], xb = sb[tt] * vj;
#pragma unroll
        for (int i = 0; i < R; ++i) Sj[i] = a * Sj[i] + xb * kr[i];
        o = 0.f;
      }
      if (readout && rp == 0) so[tt][j * kCols + cl] = o;
      }
    };
    if (ST > 1 && nt == ST) {
#pragma unroll 4
      for (int tt = 0; tt < ST; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) token(tt);
    }
    prev_t0 = t0;
    prev_nt = nt;
  }
  __syncthreads();
  if (mode != 1 && cl < prev_nt) {
#pragma unroll
    for (int j = 0; j < CG; ++j)
      if (c0 + j * kCols + rp < dv)
        p.out[static_cast<long>(row0 + prev_t0 + cl) * HV + hd * dv + c0 + j * kCols + rp] = so[cl][j * kCols + rp];
  }
  if (!DELTA && mode == 1 && blockIdx.x == 0) {  // the piece's decay: exp(-sum) carries a state across it
    if (rp == 0) sa[cl] = dsum;
    __syncthreads();
    if (tid == 0) {
      float t = 0.f;
      for (int i = 0; i < kST; ++i) t += sa[i];
      p.sc_decay[(static_cast<long>(s) * np + pc) * H + hd] = t;
    }
  }
  if (write_state) {
#pragma unroll
    for (int j = 0; j < CG; ++j) {
      const int col = c0 + j * kCols + cl;
      if (col >= out_cols) continue;
      float* Sg = Sout0 + (static_cast<long>(hd) * out_cols + col) * dk + rp * R;
      if (run_in) {
        store_run<R>(Sg, S[j], flags & 8);
      } else {
#pragma unroll
        for (int i = 0; i < R; ++i)
          if (rp * R + i < dk) Sg[i] = S[j][i];
      }
    }
  }
}

// Chains the pieces of a split state-space scan: sc_start[s][p] = the state at the start of piece p, from
// the slot (or zero for a sequence's first tokens), the pieces' end states from an empty state and
// their decays.  One thread per state element, pieces walked in order.
__global__ void __launch_bounds__(256) column_chain_kernel(const ScanArgs p) {
  const int s = blockIdx.x, hd = blockIdx.y;
  const long per_head = static_cast<long>(p.dv) * p.dk;
  const long e = static_cast<long>(blockIdx.z) * 256 + threadIdx.x;
  if (e >= per_head) return;
  const int row0 = p.qsl[s];
  if (row0 < 0 || row0 >= p.n_rows) return;
  const int qlen = min(p.qsl[s + 1], p.n_rows) - row0;
  if (qlen <= 0) return;
  const int np = min((qlen + p.piece - 1) / p.piece, p.npieces);
  const long at = hd * per_head + e, all = static_cast<long>(p.H) * per_head;
  const float* slot = p.state + static_cast<long>(p.state_rows[s]) * p.state_stride + p.off;
  float cur = p.seq_lens[s] - qlen <= 0 ? 0.f : slot[at];
  for (int pc = 0; pc < np; ++pc) {
    const long sc = (static_cast<long>(s) * p.npieces + pc) * all + at;
    p.sc_start[sc] = cur;
    if (pc == np - 1) break;
    cur = expf(-p.sc_decay[(static_cast<long>(s) * p.npieces + pc) * p.H + hd]) * cur + p.sc_local[sc];
  }
}

template <typename T, bool DELTA>
static bool launch_cs(const ScanArgs& a, int S, hipStream_t st) {
  const int ncols = (DELTA && a.mode == 1) ? a.dv + a.dk : a.dv;
  const int wc = a.max_q == 1 ? 4 * kCols : kCols;  // columns per workgroup
  const dim3 grid((ncols + wc - 1) / wc, a.H, S * a.npieces), block(256);
  if (grid.z > 65535u) return false;
  const int R = a.dk <= 32 ? 2 : a.dk <= 64 ? 4 : a.dk <= 128 ? 8 : 16;
  // which operands' runs of R elements are aligned to their size (16 bytes at most): 1 k, 2 q, 4 a, 8 state
  const size_t es = sizeof(T), al = std::min<size_t>(16, R * es), sal = std::min<size_t>(16, R * 4);
  auto ok = [&](const void* ptr, long stride) {
    return ptr != nullptr && reinterpret_cast<uintptr_t>(ptr) % al == 0 && (stride * es) % al == 0 && (a.dk * es) % al == 0;
  };
  int flags = (ok(a.k, a.k_stride) ? 1 : 0) | (ok(a.q, a.q_stride) ? 2 : 0) | (DELTA && ok(a.a, a.a_stride) ? 4 : 0);
  if (reinterpret_cast<uintptr_t>(a.state) % sal == 0 && (a.state_stride * 4) % sal == 0 && (a.off * 4) % sal == 0 &&
      (a.dk * 4) % sal == 0)
    flags |= 8;
#define MIX_CS(R)                                                                                              \
  do {                                                                                                         \
    if (a.max_q == 1) hipLaunchKernelGGL((column_scan_kernel<T, R, DELTA, 1, 4>), grid, block, 0, st, a, flags);  \
    else hipLaunchKernelGGL((column_scan_kernel<T, R, DELTA, kST, 1>), grid, block, 0, st, a, flags);             \
  } while (0)
  if (a.dk <= 32) MIX_CS(2);
  else if (a.dk <= 64) MIX_CS(4);
  else if (a.dk <= 128) MIX_CS(8);
  else if (a.dk <= 256) MIX_CS(16);
  else return false;
#undef MIX_CS
  MXS_CHECK_LAUNCH();
  return true;
}

static bool launch_pass(const ScanArgs& a, int S, bool delta, bool bf, hipStream_t st) {
  if (bf) return delta ? launch_cs<bf16_t, true>(a, S, st) : launch_cs<bf16_t, false>(a, S, st);
  return delta ? launch_cs<float, true>(a, S, st) : launch_cs<float, false>(a, S, st);
}

bool launch_column_scan(const ScanArgs& a0, int S, bool delta, bool bf, hipStream_t st) {
  if (S == 0 || a0.n_rows == 0) return true;
  ScanArgs a = a0;
  if (a.npieces <= 1) {
    a.mode = 0;
    a.piece = 1;
    a.npieces = 1;
    return launch_pass(a, S, delta, bf, st);
  }
  // the delta rule's step is no diagonal map of the state: the caller runs its passes one by one and
  // chains the pieces with matrix products in between (mxserve/ops/seqmix.py delta_scan)
  if (delta) return (a.mode == 1 || a.mode == 2) && launch_pass(a, S, true, bf, st);
  a.mode = 1;
  if (!launch_pass(a, S, false, bf, st)) return false;
  const long per_head = static_cast<long>(a.dv) * a.dk;
  hipLaunchKernelGGL(column_chain_kernel, dim3(S, a.H, static_cast<unsigned>((per_head + 255) / 256)), dim3(256), 0, st, a);
  MXS_CHECK_LAUNCH();
  a.mode = 2;
  return launch_pass(a, S, false, bf, st);
}

}  // namespace mxs
