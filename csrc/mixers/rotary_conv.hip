// Kernels around rotary attention, short causal convolutions and gated output norms (gfx950):
// scaled embedding rows into the fp32 stream, SiLU(gate) * up, q/k head norm + rotary pairs + paged
// cache write in one launch, turning attention outputs back, the convolution with its carried
// inputs, and the norm of a recurrent mixer's read-out with its gate.  Activations and weights are
// bf16 or fp32; angles, norms, sums and activations are fp32 with one rounding at the store.
#include "mix_common.h"

namespace mxs {

__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

template <typename T>
__global__ void __launch_bounds__(256) embed_scaled_kernel(float* __restrict__ out, const int64_t* __restrict__ ids,
                                                           const T* __restrict__ table, int W, long vocab, float scale) {
  const long row = blockIdx.x;
  int64_t id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // never outside the table, whatever the batch holds
  for (int c = threadIdx.x; c < W; c += blockDim.x) out[row * W + c] = ldf(table + id * W + c) * scale;
}

template <typename T>
__global__ void __launch_bounds__(256) silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, long gu_stride,
                                                       int F, long n) {
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < n; i += static_cast<long>(gridDim.x) * blockDim.x) {
    const long t = i / F;
    const int c = static_cast<int>(i - t * F);
    const T* r = gu + t * gu_stride;
    stf(out + i, silu_f(ldf(r + c)) * ldf(r + F + c));
  }
}

// One wave per (token, head): optional RMS norm over the head, interleaved rotary pairs (2i, 2i+1) on
// the first 2*nf dimensions, one store.  The grid's heads are the H query heads (rewritten in place),
// then G key heads and G value heads (into the paged cache; values have no norm and their own
// frequencies, possibly none).
template <typename T>
__global__ void __launch_bounds__(64) rope_qkv_cache_kernel(
    T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride,
    const int64_t* __restrict__ positions, const int64_t* __restrict__ slots, T* __restrict__ cache, long block_stride,
    int koff, int voff, int H, int G, int dk, int dv, int bs, const float* __restrict__ freqs, int nf,
    const T* __restrict__ q_norm, const T* __restrict__ k_norm, float eps, const float* __restrict__ v_freqs, int nvf) {
  const long t = blockIdx.x;
  const int hy = blockIdx.y, lane = threadIdx.x;
  const T* src;
  T* dst;
  const T* nw = nullptr;
  const float* fr = freqs;
  int dim = dk, nfr = nf;
  if (hy < H) {
    dst = q + t * q_stride + static_cast<long>(hy) * dk;
    src = dst;
    nw = q_norm;
  } else {
    const int64_t slot = slots[t];
    if (slot < 0) return;
    const long blk = slot / bs;
    const int off = static_cast<int>(slot % bs);
    if (hy < H + G) {
      const int g = hy - H;
      src = k + t * k_stride + static_cast<long>(g) * dk;
      dst = cache + blk * block_stride + koff + (static_cast<long>(g) * bs + off) * dk;
      nw = k_norm;
    } else {
      const int g = hy - H - G;
      src = v + t * v_stride + static_cast<long>(g) * dv;
      dst = cache + blk * block_stride + voff + (static_cast<long>(g) * bs + off) * dv;
      dim = dv;
      fr = v_freqs;
      nfr = nvf;
    }
  }
  float inv = 1.f;
  if (nw != nullptr) {
    float s = 0.f;
    for (int d = lane; d < dim; d += 64) { const float x = ldf(src + d); s += x * x; }
    inv = rsqrtf(wave_sum(s) / static_cast<float>(dim) + eps);
  }
  const float pos = static_cast<float>(positions[t]);
  for (int pr = lane; 2 * pr < dim; pr += 64) {
    const int d0 = 2 * pr;
    const bool two = d0 + 1 < dim;
    float a = ldf(src + d0) * inv, b = two ? ldf(src + d0 + 1) * inv : 0.f;
    if (nw != nullptr) { a *= ldf(nw + d0); if (two) b *= ldf(nw + d0 + 1); }
    if (pr < nfr) {
      float sn, cs;
      sincosf(pos * fr[pr], &sn, &cs);
      const float a2 = a * cs - b * sn;
      b = b * cs + a * sn;
      a = a2;
    }
    stf(dst + d0, a);
    if (two) stf(dst + d0 + 1, b);
  }
}

// out = scale * (x with the pairs of every head turned by sign * position * freqs); out rows may be
// a slice of a wider buffer.
template <typename T>
__global__ void __launch_bounds__(64) rope_rows_kernel(T* __restrict__ out, long out_stride, const T* __restrict__ x,
                                                       long x_stride, const int64_t* __restrict__ positions, int dim,
                                                       const float* __restrict__ freqs, int nf, float sign, float scale) {
  const long t = blockIdx.x;
  const int hd = blockIdx.y, lane = threadIdx.x;
  const T* src = x + t * x_stride + static_cast<long>(hd) * dim;
  T* dst = out + t * out_stride + static_cast<long>(hd) * dim;
  const float pos = static_cast<float>(positions[t]) * sign;
  for (int pr = lane; 2 * pr < dim; pr += 64) {
    const int d0 = 2 * pr;
    const bool two = d0 + 1 < dim;
    float a = ldf(src + d0), b = two ? ldf(src + d0 + 1) : 0.f;
    if (pr < nf) {
      float sn, cs;
      sincosf(pos * freqs[pr], &sn, &cs);
      const float a2 = a * cs - b * sn;
      b = b * cs + a * sn;
      a = a2;
    }
    stf(dst + d0, a * scale);
    if (two) stf(dst + d0 + 1, b * scale);
  }
}

// y[t, c] = act(bias[c] + sum_j w[j, c] x[t - (taps-1) + j, c]), w tap-major [taps, C]; inputs before the
// chunk come from the sequence's state rows [taps-1, C] (oldest first), zeros for a sequence's first
// tokens.  A thread takes V consecutive channels: V = 16 bytes' worth when rows, weights and channel
// count allow whole 16-byte pieces, else 1.
template <typename T> struct Piece;
template <> struct Piece<bf16_t> { static constexpr int N = 8; };
template <> struct Piece<float> { static constexpr int N = 4; };
__device__ __forceinline__ void load_piece(const bf16_t* p, float* o) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  o[0] = bf2f_lo(a.x); o[1] = bf2f_hi(a.x); o[2] = bf2f_lo(a.y); o[3] = bf2f_hi(a.y);
  o[4] = bf2f_lo(a.z); o[5] = bf2f_hi(a.z); o[6] = bf2f_lo(a.w); o[7] = bf2f_hi(a.w);
}
__device__ __forceinline__ void load_piece(const float* p, float* o) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void store_piece(bf16_t* p, const float* o) {
  uint4 a;
  a.x = pack2(o[0], o[1]); a.y = pack2(o[2], o[3]); a.z = pack2(o[4], o[5]); a.w = pack2(o[6], o[7]);
  *reinterpret_cast<uint4*>(p) = a;
}
__device__ __forceinline__ void store_piece(float* p, const float* o) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}

template <typename T, bool WIDE>
__global__ void __launch_bounds__(256) causal_conv_kernel(T* __restrict__ out, const T* __restrict__ x, long x_stride,
                                                          const T* __restrict__ w, const T* __restrict__ bias,
                                                          const float* __restrict__ state, long state_stride,
                                                          const int* __restrict__ state_rows, long off,
                                                          const int* __restrict__ qsl, const int* __restrict__ seq_lens,
                                                          int S, int C, int taps, int silu) {
  constexpr int V = WIDE ? Piece<T>::N : 1;
  const int t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * V;
  if (c >= C) return;
  const int s = seq_of_row(qsl, S, t);
  const int row0 = qsl[s], qlen = qsl[s + 1] - row0;
  const int i = t - row0;
  const bool fresh = seq_lens[s] - qlen <= 0;
  const float* st = state + static_cast<long>(state_rows[s]) * state_stride + off;
  float acc[V], xv[V], wv[V];
  if constexpr (WIDE) {
    if (bias) load_piece(bias + c, acc);
    else for (int e = 0; e < V; ++e) acc[e] = 0.f;
  } else {
    acc[0] = bias ? ldf(bias + c) : 0.f;
  }
  for (int j = 0; j < taps; ++j) {
    const int src = i - (taps - 1 - j);
    if (src < 0 && fresh) continue;
    if constexpr (WIDE) {
      if (src >= 0) {
        load_piece(x + static_cast<long>(row0 + src) * x_stride + c, xv);
      } else {
        const float* sp = st + static_cast<long>(taps - 1 + src) * C + c;
#pragma unroll
        for (int e = 0; e < V; e += 4) load_piece(sp + e, xv + e);
      }
      load_piece(w + static_cast<long>(j) * C + c, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += wv[e] * xv[e];
    } else {
      xv[0] = src >= 0 ? ldf(x + static_cast<long>(row0 + src) * x_stride + c) : st[static_cast<long>(taps - 1 + src) * C + c];
      acc[0] += ldf(w + static_cast<long>(j) * C + c) * xv[0];
    }
  }
  if (silu) {
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = silu_f(acc[e]);
  }
  if constexpr (WIDE) store_piece(out + static_cast<long>(t) * C + c, acc);
  else stf(out + static_cast<long>(t) * C + c, acc[0]);
}

// The state after the step: the last taps-1 inputs of (old state ++ chunk).  Row r of the new state
// reads old row r + n or a chunk row, so one thread per channel walking r upwards never reads what it
// has already replaced.  Runs after causal_conv_kernel on the same stream.
template <typename T>
__global__ void __launch_bounds__(256) conv_state_kernel(const T* __restrict__ x, long x_stride, float* __restrict__ state,
                                                         long state_stride, const int* __restrict__ state_rows, long off,
                                                         const int* __restrict__ qsl, const int* __restrict__ seq_lens,
                                                         int n_rows, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int row0 = qsl[s];
  if (row0 < 0 || row0 >= n_rows) return;
  const int n = min(qsl[s + 1], n_rows) - row0;
  if (n <= 0) return;
  const bool fresh = seq_lens[s] - n <= 0;
  float* st = state + static_cast<long>(state_rows[s]) * state_stride + off;
  for (int r = 0; r < taps - 1; ++r) {
    const int src = n - (taps - 1) + r;
    float xv = 0.f;
    if (src >= 0) xv = ldf(x + static_cast<long>(row0 + src) * x_stride + c);
    else if (!fresh) xv = st[static_cast<long>(taps - 1 + src) * C + c];
    st[static_cast<long>(r) * C + c] = xv;
  }
}

// out = scale * [ RMSNorm_groups(o * act(gate)) * w ]            (gate_first)
//     = scale * [ RMSNorm_groups(o) * w * act(gate) ]            (otherwise)
// act = SiLU or sigmoid; w repeats with period wn; one wave per slice of the row (groups > 1) or the
// block for the whole row.
template <typename T>
__global__ void __launch_bounds__(256) gated_norm_kernel(T* __restrict__ out, long out_stride, const float* __restrict__ o,
                                                         const T* __restrict__ gate, long g_stride,
                                                         const T* __restrict__ w, int wn, int N, int groups, float eps,
                                                         int silu, int gate_first, float scale) {
  __shared__ float scratch[16];
  const long row = blockIdx.x;
  const float* orow = o + row * N;
  const T* grow = gate + row * g_stride;
  T* yrow = out + row * out_stride;
  auto act = [&](int c) { const float z = ldf(grow + c); return silu ? silu_f(z) : sigmoid_f(z); };
  if (groups == 1) {
    float s = 0.f;
    for (int c = threadIdx.x; c < N; c += blockDim.x) {
      const float v = gate_first ? orow[c] * act(c) : orow[c];
      s += v * v;
    }
    const float inv = rsqrtf(block_sum(s, scratch) / static_cast<float>(N) + eps);
    for (int c = threadIdx.x; c < N; c += blockDim.x)
      stf(yrow + c, orow[c] * act(c) * inv * ldf(w + c % wn) * scale);
    return;
  }
  const int n = N / groups, lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int g = wid; g < groups; g += nw) {
    float s = 0.f;
    for (int c = lane; c < n; c += 64) {
      const int i = g * n + c;
      const float v = gate_first ? orow[i] * act(i) : orow[i];
      s += v * v;
    }
    const float inv = rsqrtf(wave_sum(s) / static_cast<float>(n) + eps);
    for (int c = lane; c < n; c += 64) {
      const int i = g * n + c;
      stf(yrow + i, orow[i] * act(i) * inv * ldf(w + i % wn) * scale);
    }
  }
}

#define MIX_DISPATCH(bf, ...)                      \
  do {                                             \
    if (bf) { using T = bf16_t; __VA_ARGS__; }     \
    else { using T = float; __VA_ARGS__; }         \
  } while (0)

void launch_embed_scaled(float* out, const int64_t* ids, const void* table, int rows, int W, long vocab, float scale,
                         bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(embed_scaled_kernel<T>, dim3(rows), dim3(256), 0, st, out, ids, (const T*)table, W,
                                      vocab, scale));
  MXS_CHECK_LAUNCH();
}

void launch_silu_mul(void* out, const void* gu, long gu_stride, int rows, int F, bool bf, hipStream_t st) {
  const long n = static_cast<long>(rows) * F;
  if (n == 0) return;
  const int blocks = static_cast<int>(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
  MIX_DISPATCH(bf, hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, st, (T*)out, (const T*)gu, gu_stride,
                                      F, n));
  MXS_CHECK_LAUNCH();
}

void launch_rope_qkv_cache(void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                           const int64_t* positions, const int64_t* slots, void* cache, long block_stride, int rows,
                           int koff, int voff, int H, int G, int dk, int dv, int bs, const float* freqs, int nf,
                           const void* q_norm, const void* k_norm, float eps, const float* v_freqs, int nvf, bool bf,
                           hipStream_t st) {
  if (rows == 0) return;
  const dim3 grid(rows, H + (k != nullptr ? 2 * G : 0));
  MIX_DISPATCH(bf, hipLaunchKernelGGL(rope_qkv_cache_kernel<T>, grid, dim3(64), 0, st, (T*)q, q_stride, (const T*)k,
                                      k_stride, (const T*)v, v_stride, positions, slots, (T*)cache, block_stride, koff,
                                      voff, H, G, dk, dv, bs, freqs, nf, (const T*)q_norm, (const T*)k_norm, eps, v_freqs,
                                      nvf));
  MXS_CHECK_LAUNCH();
}

void launch_rope_rows(void* out, long out_stride, const void* x, long x_stride, const int64_t* positions, int rows,
                      int heads, int dim, const float* freqs, int nf, float sign, float scale, bool bf, hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(rope_rows_kernel<T>, dim3(rows, heads), dim3(64), 0, st, (T*)out, out_stride,
                                      (const T*)x, x_stride, positions, dim, freqs, nf, sign, scale));
  MXS_CHECK_LAUNCH();
}

void launch_causal_conv(void* out, const void* x, long x_stride, const void* w, const void* bias, float* state,
                        long state_stride, const int* state_rows, long off, const int* qsl, const int* seq_lens, int S,
                        int rows, int C, int taps, int silu, bool bf, hipStream_t st) {
  if (rows == 0 || S == 0) return;
  const int cb = (C + 255) / 256;
  // whole 16-byte pieces everywhere: rows, weights, bias, output, and the fp32 state rows
  const int v = bf ? 8 : 4;
  auto al = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
  const bool wide = C % v == 0 && x_stride % v == 0 && al(x) && al(w) && al(out) && (bias == nullptr || al(bias)) &&
                    al(state) && state_stride % 4 == 0 && off % 4 == 0;
  if (wide) {
    const int cw = (C / v + 255) / 256;
    MIX_DISPATCH(bf, hipLaunchKernelGGL((causal_conv_kernel<T, true>), dim3(rows, cw), dim3(256), 0, st, (T*)out,
                                        (const T*)x, x_stride, (const T*)w, (const T*)bias, state, state_stride,
                                        state_rows, off, qsl, seq_lens, S, C, taps, silu));
  } else {
    MIX_DISPATCH(bf, hipLaunchKernelGGL((causal_conv_kernel<T, false>), dim3(rows, cb), dim3(256), 0, st, (T*)out,
                                        (const T*)x, x_stride, (const T*)w, (const T*)bias, state, state_stride,
                                        state_rows, off, qsl, seq_lens, S, C, taps, silu));
  }
  MXS_CHECK_LAUNCH();
  if (taps > 1) {
    MIX_DISPATCH(bf, hipLaunchKernelGGL(conv_state_kernel<T>, dim3(S, cb), dim3(256), 0, st, (const T*)x, x_stride, state,
                                        state_stride, state_rows, off, qsl, seq_lens, rows, C, taps));
    MXS_CHECK_LAUNCH();
  }
}

void launch_gated_norm(void* out, long out_stride, const float* o, const void* gate, long g_stride, const void* w, int wn,
                       int rows, int N, int groups, float eps, int silu, int gate_first, float scale, bool bf,
                       hipStream_t st) {
  if (rows == 0) return;
  MIX_DISPATCH(bf, hipLaunchKernelGGL(gated_norm_kernel<T>, dim3(rows), dim3(256), 0, st, (T*)out, out_stride, o,
                                      (const T*)gate, g_stride, (const T*)w, wn, N, groups, eps, silu, gate_first, scale));
  MXS_CHECK_LAUNCH();
}

}  // namespace mxs
