// torch bindings of the mixer kernels (mxserve/_M): shape and dtype checks on the host, so that a
// launch never reads or writes outside what the kernels and their grids assume.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>
#include <torch/extension.h>

namespace mxs {
void launch_resid_update(float*, const void*, long, const void*, const void*, long, const void*, const void*, int,
                         const void*, void*, int, int, float, bool, hipStream_t);
void launch_cast_into(void*, long, const float*, int, int, bool, hipStream_t);
void launch_relu_sq(void*, const void*, long, bool, hipStream_t);
void launch_softcap(float*, const void*, long, int, int, float, bool, hipStream_t);
void launch_gated_rms_norm(void*, const float*, const void*, long, const void*, int, int, int, float, bool, hipStream_t);
void launch_gate_linear(float*, const void*, long, const void*, const void*, int, int, int, bool, hipStream_t);
void launch_kv_write(void*, long, const void*, long, const void*, long, const int64_t*, int, int, int, int, int, int,
                     int, bool, hipStream_t);
bool launch_window_attention(void*, const void*, long, const void*, long, const int*, int, const int*, const int*, int,
                             int, int, int, int, int, int, int, int, float, int, int, int, bool, hipStream_t);
bool launch_matrix_scan(float*, const void*, long, const void*, long, const void*, long, const float*, const float*,
                        float*, long, const int*, long, const int*, const int*, int, int, int, int, int, int, float,
                        float, bool, bool, int, int, float*, float*, long, hipStream_t);
}  // namespace mxs

namespace {

using OptT = c10::optional<at::Tensor>;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_bf(const at::Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, "activations must be bf16 or fp32");
  return t.scalar_type() == at::kBFloat16;
}

// a [rows, cols] matrix of dtype `bf`, unit column stride
const void* mat(const at::Tensor& t, bool bf, int64_t rows, int64_t cols, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.size(0) == rows && t.size(1) == cols && (cols == 1 || t.stride(1) == 1),
              name, ": expected a GPU [", rows, ", ", cols, "] matrix with contiguous rows");
  TORCH_CHECK(is_bf(t) == bf, name, ": dtype differs from the other operands");
  return t.data_ptr();
}

const void* vec(const OptT& t, bool bf, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->numel() == n, name, ": expected ", n, " contiguous elements");
  TORCH_CHECK(is_bf(*t) == bf, name, ": dtype differs from the other operands");
  return t->data_ptr();
}

const int* i32(const at::Tensor& t, int64_t n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous() && t.numel() >= n, name,
              ": expected >= ", n, " contiguous int32");
  return t.data_ptr<int>();
}

float* f32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, ": expected contiguous fp32");
  return t.data_ptr<float>();
}

void resid_update(at::Tensor x, OptT a, OptT wa, OptT b, OptT wb, OptT bias, bool assign, OptT norm_w, OptT h,
                  double eps) {
  float* xp = f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x: [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const at::Tensor* any = a.has_value() ? &*a : (norm_w.has_value() ? &*norm_w : nullptr);
  if (any == nullptr || T == 0) return;
  const bool bf = is_bf(*any);
  const void* ap = a.has_value() ? mat(*a, bf, T, W, "a") : nullptr;
  const void* bp = b.has_value() ? mat(*b, bf, T, W, "b") : nullptr;
  TORCH_CHECK(!b.has_value() || (a.has_value() && wa.has_value() && wb.has_value()), "two branches need both weights");
  TORCH_CHECK(!assign || a.has_value(), "assign needs a");
  TORCH_CHECK(norm_w.has_value() == h.has_value(), "norm_w and h go together");
  void* hp = nullptr;
  if (h.has_value()) {
    TORCH_CHECK(h->is_cuda() && h->is_contiguous() && h->dim() == 2 && h->size(0) == T && h->size(1) == W &&
                is_bf(*h) == bf, "h: contiguous [T, W] of the operands' dtype");
    hp = h->data_ptr();
  }
  mxs::launch_resid_update(xp, ap, a.has_value() ? a->stride(0) : 0, vec(wa, bf, W, "wa"), bp,
                           b.has_value() ? b->stride(0) : 0, vec(wb, bf, W, "wb"), vec(bias, bf, W, "bias"), assign,
                           vec(norm_w, bf, W, "norm_w"), hp, static_cast<int>(T), static_cast<int>(W),
                           static_cast<float>(eps), bf, stream());
}

void cast_into(at::Tensor dst, at::Tensor x) {
  const float* xp = f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && dst.is_cuda() && dst.dim() == 2 && dst.size(0) == x.size(0) && dst.size(1) >= x.size(1) &&
              dst.stride(1) == 1, "dst: [T, >= W] with contiguous rows");
  mxs::launch_cast_into(dst.data_ptr(), dst.stride(0), xp, static_cast<int>(x.size(0)), static_cast<int>(x.size(1)),
                        is_bf(dst), stream());
}

void relu_sq(at::Tensor out, at::Tensor x) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous() && out.is_contiguous() && out.numel() == x.numel() &&
              out.scalar_type() == x.scalar_type(), "relu_sq: contiguous tensors of one dtype");
  mxs::launch_relu_sq(out.data_ptr(), x.data_ptr(), x.numel(), is_bf(x), stream());
}

void softcap(at::Tensor out, at::Tensor x, double cap) {
  float* op = f32(out, "out");
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 && out.dim() == 2 && out.size(0) == x.size(0) &&
              out.size(1) == x.size(1), "softcap: [n, V]");
  mxs::launch_softcap(op, x.data_ptr(), x.stride(0), static_cast<int>(x.size(0)), static_cast<int>(x.size(1)),
                      static_cast<float>(cap), is_bf(x), stream());
}

void gated_rms_norm(at::Tensor out, at::Tensor o, at::Tensor gate, at::Tensor w, double eps, int64_t groups) {
  const float* opn = f32(o, "o");
  TORCH_CHECK(o.dim() == 2, "o: [T, N]");
  const int64_t T = o.size(0), N = o.size(1);
  const bool bf = is_bf(out);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == N, "out: [T, N]");
  TORCH_CHECK(groups >= 1 && N % groups == 0, "groups must divide N");
  mxs::launch_gated_rms_norm(out.data_ptr(), opn, mat(gate, bf, T, N, "gate"), gate.stride(0), vec(OptT(w), bf, N, "w"),
                             static_cast<int>(T), static_cast<int>(N), static_cast<int>(groups), static_cast<float>(eps),
                             bf, stream());
}

void gate_linear(at::Tensor out, at::Tensor h, at::Tensor w, OptT bias) {
  float* op = f32(out, "out");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.stride(1) == 1 && w.is_cuda() && w.dim() == 2 && w.is_contiguous() &&
              w.size(1) == h.size(1) && out.dim() == 2 && out.size(0) == h.size(0) && out.size(1) == w.size(0),
              "gate_linear: h [T, W], w [N, W], out [T, N]");
  const bool bf = is_bf(h);
  TORCH_CHECK(is_bf(w) == bf, "w: dtype differs from h");
  mxs::launch_gate_linear(op, h.data_ptr(), h.stride(0), w.data_ptr(), vec(bias, bf, w.size(0), "bias"),
                          static_cast<int>(h.size(0)), static_cast<int>(w.size(0)), static_cast<int>(w.size(1)), bf,
                          stream());
}

void check_cache(const at::Tensor& cache, bool bf, int64_t koff, int64_t voff, int64_t G, int64_t dk, int64_t dv,
                 int64_t bs) {
  TORCH_CHECK(cache.is_cuda() && cache.dim() == 2 && cache.is_contiguous() && is_bf(cache) == bf,
              "cache: contiguous [blocks, block_elems] of the operands' dtype");
  TORCH_CHECK(koff >= 0 && voff >= 0 && koff + G * bs * dk <= cache.size(1) && voff + G * bs * dv <= cache.size(1),
              "K/V region outside a cache block");
}

void kv_write(at::Tensor cache, at::Tensor k, at::Tensor v, at::Tensor slots, int64_t koff, int64_t voff, int64_t G,
              int64_t dk, int64_t dv, int64_t bs) {
  const bool bf = is_bf(k);
  const int64_t T = k.size(0);
  check_cache(cache, bf, koff, voff, G, dk, dv, bs);
  TORCH_CHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T,
              "slot_mapping: int64 [T]");
  mxs::launch_kv_write(cache.data_ptr(), cache.stride(0), mat(k, bf, T, G * dk, "k"), k.stride(0),
                       mat(v, bf, T, G * dv, "v"), v.stride(0), slots.data_ptr<int64_t>(), static_cast<int>(T),
                       static_cast<int>(koff), static_cast<int>(voff), static_cast<int>(G), static_cast<int>(dk),
                       static_cast<int>(dv), static_cast<int>(bs), bf, stream());
}

void window_attention(at::Tensor out, at::Tensor q, at::Tensor cache, at::Tensor block_tables, at::Tensor qsl,
                      at::Tensor seq_lens, int64_t koff, int64_t voff, int64_t H, int64_t G, int64_t dk, int64_t dv,
                      int64_t bs, double scale, int64_t window, int64_t keep, int64_t max_query_len) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0), S = seq_lens.numel();
  check_cache(cache, bf, koff, voff, G, dk, dv, bs);
  TORCH_CHECK(G >= 1 && H % G == 0, "query heads must divide over kv heads");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv &&
              is_bf(out) == bf, "out: [T, H*dv]");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
              block_tables.size(0) >= S && block_tables.stride(1) == 1, "block_tables: int32 [S, max_blocks]");
  const bool ok = mxs::launch_window_attention(
      out.data_ptr(), mat(q, bf, T, H * dk, "q"), q.stride(0), cache.data_ptr(), cache.stride(0),
      block_tables.data_ptr<int>(), static_cast<int>(block_tables.stride(0)), i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(koff),
      static_cast<int>(voff), static_cast<int>(H), static_cast<int>(G), static_cast<int>(dk), static_cast<int>(dv),
      static_cast<int>(bs), static_cast<float>(scale), static_cast<int>(window), static_cast<int>(keep),
      static_cast<int>(std::min<int64_t>(max_query_len, T)), bf, stream());
  TORCH_CHECK(ok, "window_attention: head sizes beyond what the kernel holds (dv <= 512)");
}

void scan(bool mlstm, at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, const float* decay, const float* gates,
          at::Tensor state, at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H,
          int64_t dk, int64_t dv, bool silu, double cap, double q_scale, int64_t piece, int64_t npieces, OptT sc_local,
          OptT sc_start) {
  const bool bf = is_bf(q);
  const int64_t T = q.size(0), S = seq_lens.numel();
  float* op = f32(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv, "out: fp32 [T, H*dv]");
  float* sp = f32(state, "state");
  const int64_t need = mlstm ? H * (dk * dv + dk + 1) : H * dk * dv;
  TORCH_CHECK(state.dim() == 2 && off >= 0 && off + need <= state.size(1), "state slot too small for this layer");
  // time-split launches: two scratch pools of [S, npieces, sc_floats] (a piece's end state; mLSTM: plus [H] sums)
  const int64_t sc_floats = need + (mlstm ? H : 0);
  float *scl = nullptr, *scs = nullptr;
  if (npieces > 1) {
    TORCH_CHECK(piece >= 16 && sc_local.has_value() && sc_start.has_value(), "a split scan needs its scratch pools");
    scl = f32(*sc_local, "sc_local");
    scs = f32(*sc_start, "sc_start");
    TORCH_CHECK(sc_local->numel() >= S * npieces * sc_floats && sc_start->numel() >= S * npieces * sc_floats,
                "scratch pools smaller than [S, npieces, state]");
  } else {
    piece = 1;
    npieces = 1;
  }
  const bool ok = mxs::launch_matrix_scan(
      op, mat(q, bf, T, H * dk, "q"), q.stride(0), mat(k, bf, T, H * dk, "k"), k.stride(0), mat(v, bf, T, H * dv, "v"),
      v.stride(0), decay, gates, sp, state.stride(0), i32(state_rows, S, "state_rows"), off, i32(qsl, S + 1, "qsl"),
      i32(seq_lens, S, "seq_lens"), static_cast<int>(S), static_cast<int>(T), static_cast<int>(H), static_cast<int>(dk),
      static_cast<int>(dv), silu ? 1 : 0, static_cast<float>(cap), static_cast<float>(q_scale), mlstm, bf,
      static_cast<int>(piece), static_cast<int>(npieces), scl, scs, sc_floats, stream());
  TORCH_CHECK(ok, "matrix scan: key size beyond 256");
}

void decay_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor decay, at::Tensor state,
                at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H, int64_t dk,
                int64_t dv, bool silu, int64_t piece, int64_t npieces, OptT sc_local, OptT sc_start) {
  TORCH_CHECK(decay.numel() == H, "decay: fp32 [H]");
  scan(false, out, q, k, v, f32(decay, "decay"), nullptr, state, state_rows, off, qsl, seq_lens, H, dk, dv, silu, 0.0, 1.0,
       piece, npieces, sc_local, sc_start);
}

void mlstm_scan(at::Tensor out, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor gates, at::Tensor state,
                at::Tensor state_rows, int64_t off, at::Tensor qsl, at::Tensor seq_lens, int64_t H, int64_t dk,
                int64_t dv, double cap, double q_scale, int64_t piece, int64_t npieces, OptT sc_local, OptT sc_start) {
  TORCH_CHECK(gates.dim() == 2 && gates.size(0) == q.size(0) && gates.size(1) == 2 * H, "gates: fp32 [T, 2H]");
  scan(true, out, q, k, v, nullptr, f32(gates, "gates"), state, state_rows, off, qsl, seq_lens, H, dk, dv, false, cap,
       q_scale, piece, npieces, sc_local, sc_start);
}

}  // namespace

PYBIND11_MODULE(_M, m) {
  m.def("resid_update", &resid_update);
  m.def("cast_into", &cast_into);
  m.def("relu_sq", &relu_sq);
  m.def("softcap", &softcap);
  m.def("gated_rms_norm", &gated_rms_norm);
  m.def("gate_linear", &gate_linear);
  m.def("kv_write", &kv_write);
  m.def("window_attention", &window_attention);
  m.def("decay_scan", &decay_scan);
  m.def("mlstm_scan", &mlstm_scan);
}
