// Softmax attention over the paged cache with a sliding window and kept first tokens (gfx950),
// for prompt chunks and single decoded tokens alike: one workgroup per (query row, query head).
// The query at position i sees key j <= i when i - j < window or j < keep (window <= 0: all j <= i).
// Visible keys are walked in tiles of 256: one key per thread for the scores (fp32 dot of the LDS
// query with the key's cache row), a block-wide running maximum and sum (online softmax), then each
// wave takes every fourth key of the tile with its lanes across the value row.  Scores, weights and
// the output sum are fp32; q, K and V are bf16 or fp32.
#include "mix_common.h"

namespace mxs {

constexpr int kKeyTile = 256;
constexpr int kMaxVChunks = 8;  // value size <= 64 * 8

template <typename T>
__global__ void __launch_bounds__(256) window_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ cache, long block_stride,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    int S, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale, int window, int keep, bool vec) {
  extern __shared__ float lds[];
  float* qs = lds;                      // [dk]
  float* p = qs + ((dk + 3) & ~3);      // [kKeyTile]
  float* red = p + kKeyTile;            // [4][dv]
  __shared__ float scratch[16];
  const int t = blockIdx.x, hd = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wid = tid >> 6;
  const int s = seq_of_row(qsl, S, t);
  const int qlen = qsl[s + 1] - qsl[s];
  // the row's position, kept inside the block table whatever the metadata says
  const int pos = min(max(seq_lens[s] - qlen + (t - qsl[s]), 0), bt_stride * bs - 1);
  const int g = hd / (H / G);
  const int lo = window > 0 ? max(pos - window + 1, 0) : 0;
  const int nA = window > 0 ? min(keep, lo) : 0;  // kept first tokens that lie below the window
  const int nvis = nA + (pos - lo + 1);
  const int* bt = block_tables + static_cast<long>(s) * bt_stride;
  for (int d = tid; d < dk; d += blockDim.x) qs[d] = ldf(q + static_cast<long>(t) * q_stride + hd * dk + d) * scale;
  float m = -INFINITY, l = 0.f;
  float acc[kMaxVChunks];
#pragma unroll
  for (int c = 0; c < kMaxVChunks; ++c) acc[c] = 0.f;
  const int nchunk = (dv + 63) >> 6;
  __syncthreads();
  for (int t0 = 0; t0 < nvis; t0 += kKeyTile) {
    const int nt = min(kKeyTile, nvis - t0);
    float sc = -INFINITY;
    if (tid < nt) {
      const int n = t0 + tid;
      const int j = n < nA ? n : lo + (n - nA);
      const T* kp = cache + static_cast<long>(bt[j / bs]) * block_stride + koff + (static_cast<long>(g) * bs + j % bs) * dk;
      sc = dot_row<T>(qs, kp, dk, vec);
    }
    const float m_new = fmaxf(m, block_max(sc, scratch));
    const float e = tid < nt ? expf(sc - m_new) : 0.f;
    p[tid] = e;
    const float tsum = block_sum(e, scratch);  // its barriers also publish p
    const float corr = expf(m - m_new);        // first tile: exp(-inf) = 0, acc and l are 0
    l = l * corr + tsum;
    m = m_new;
#pragma unroll
    for (int c = 0; c < kMaxVChunks; ++c) acc[c] *= corr;
    for (int n = wid; n < nt; n += 4) {
      const int nn = t0 + n;
      const int j = nn < nA ? nn : lo + (nn - nA);
      const T* vp = cache + static_cast<long>(bt[j / bs]) * block_stride + voff + (static_cast<long>(g) * bs + j % bs) * dv;
      const float pn = p[n];
#pragma unroll
      for (int c = 0; c < kMaxVChunks; ++c) {
        const int e2 = lane + 64 * c;
        if (c < nchunk && e2 < dv) acc[c] += pn * ldf(vp + e2);
      }
    }
    __syncthreads();  // p is rewritten by the next tile
  }
#pragma unroll
  for (int c = 0; c < kMaxVChunks; ++c) {
    const int e2 = lane + 64 * c;
    if (c < nchunk && e2 < dv) red[wid * dv + e2] = acc[c];
  }
  __syncthreads();
  const float inv = 1.f / l;
  for (int e2 = tid; e2 < dv; e2 += blockDim.x) {
    const float o = red[e2] + red[dv + e2] + red[2 * dv + e2] + red[3 * dv + e2];
    stf(out + static_cast<long>(t) * (H * dv) + hd * dv + e2, o * inv);
  }
}

bool launch_window_attention(void* out, const void* q, long q_stride, const void* cache, long block_stride,
                             const int* block_tables, int bt_stride, const int* qsl, const int* seq_lens, int S,
                             int rows, int koff, int voff, int H, int G, int dk, int dv, int bs, float scale,
                             int window, int keep, bool bf, hipStream_t st) {
  if (rows == 0 || S == 0) return true;
  if (dv > 64 * kMaxVChunks) return false;
  const int el = bf ? 8 : 4;  // elements per 16-byte load
  const bool vec = dk % el == 0 && koff % el == 0 && block_stride % el == 0;
  const size_t shm = (((dk + 3) & ~3) + kKeyTile + 4 * dv) * sizeof(float);
  if (shm > 60 * 1024) return false;
  if (bf)
    hipLaunchKernelGGL(window_attention_kernel<bf16_t>, dim3(rows, H), dim3(256), shm, st, (bf16_t*)out, (const bf16_t*)q,
                       q_stride, (const bf16_t*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, koff,
                       voff, H, G, dk, dv, bs, scale, window, keep, vec);
  else
    hipLaunchKernelGGL(window_attention_kernel<float>, dim3(rows, H), dim3(256), shm, st, (float*)out, (const float*)q,
                       q_stride, (const float*)cache, block_stride, block_tables, bt_stride, qsl, seq_lens, S, koff,
                       voff, H, G, dk, dv, bs, scale, window, keep, vec);
  MXS_CHECK_LAUNCH();
  return true;
}

}  // namespace mxs
