// Python module `window_matmul_kernel` for PyTorch-ROCm: the same four functions the
// reference's native module exports (reference csrc/window_matmul/window_matmul.cpp:100-106),
// implemented as a thin layer over the C ABI in include/window_matmul_hip.h.
//
// What this layer does, and nothing more: argument checks with the reference's error
// texts (reference cuda/utils.cuh:3-4, cuda/window_matmul_cuda.cu:226-232, 323-329),
// layout normalisation, output allocation with the input's dtype and device, device
// guard, current-stream lookup, and the call into libwindow_matmul_hip.so.
//
// There is deliberately no CPU implementation behind this module: tensors that do not
// live on the GPU raise, as the reference does for GPU tensors in a CPU-only build
// (reference window_matmul.cpp:15).
#include <torch/extension.h>

#include <algorithm>
#include <stdexcept>
#include <string>
#include <vector>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>

#include "../../include/window_matmul_hip.h"

namespace {

void check_gpu(const torch::Tensor &t, const char *name) {
  TORCH_CHECK(t.device().is_cuda(), name,
              " must be CUDA tensor (window_matmul_kernel is built for MI355X only and has no CPU path)");
}

int abi_dtype(const torch::Tensor &t, const char *op) {
  switch (t.scalar_type()) {
    case at::kFloat: return WM_DTYPE_F32;
    case at::kHalf: return WM_DTYPE_F16;
    case at::kBFloat16: return WM_DTYPE_BF16;
    case at::kDouble: return WM_DTYPE_F64;
    default: TORCH_CHECK(false, "\"", op, "\" not implemented for '", c10::toString(t.scalar_type()), "'");
  }
  return -1;
}

bool aligned16(const torch::Tensor &t) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0; }

// Unit column stride and 16-byte aligned rows/batches, else a contiguous copy.
torch::Tensor vector_friendly(const torch::Tensor &t) {
  const int64_t es = t.element_size();
  const bool ok = t.stride(2) == 1 && (t.stride(1) * es) % 16 == 0 && (t.stride(0) * es) % 16 == 0 && aligned16(t);
  if (ok || t.numel() == 0) return t;
  if (t.is_contiguous()) {
    // rows that cannot be aligned (N * element size not a multiple of 16): the tile kernels take
    // the tensor as it is; alignable rows behind a misaligned pointer (a view at a storage offset)
    // move into a fresh allocation so that the tuned kernels apply
    return (t.size(2) * es) % 16 == 0 ? t.clone(at::MemoryFormat::Contiguous) : t;
  }
  auto c = t.contiguous();
  return aligned16(c) || (t.size(2) * es) % 16 != 0 ? c : c.clone(at::MemoryFormat::Contiguous);
}

// Band tensors (rows of odd length 2w+1) need to be contiguous and start on a 16-byte boundary.
torch::Tensor band_friendly(const torch::Tensor &t) {
  auto c = t.contiguous();
  return aligned16(c) || c.numel() == 0 ? c : c.clone(at::MemoryFormat::Contiguous);
}

// Head widths that the tuned kernels do not take -- N not a multiple of 16 for 16-bit storage, of 8
// for float32 -- are padded with zero columns to the next such width (up to 128): zero columns add
// nothing to a dot product and produce result columns that are cut off again, and two or three
// passes over the (B,M,N) tensors cost less than the element-by-element tile kernels, which take such
// shapes otherwise.  float64 needs none of this: its kernels take every head width.  Nor does float32
// up to w = 256, where the tile kernels were measured level with or ahead of padding and slicing
// (B96 M4096 N60: 109 against 151 us at w = 8, 184 against 245 us at w = 64; B16 M4096 N256 w256:
// 298 against 287 us; at w = 1500 the tuned kernels are 1.5 times faster again).
constexpr int64_t kTileUpToWindowF32 = 256;
bool tiles_preferred(const torch::Tensor &t, int64_t w) { return t.scalar_type() == at::kFloat && w <= kTileUpToWindowF32; }

int64_t padded_width(const torch::Tensor &t, int64_t w) {
  const int64_t N = t.size(2);
  if (tiles_preferred(t, w)) return N;
  int64_t unit;
  switch (t.scalar_type()) {
    case at::kHalf:
    case at::kBFloat16: unit = 16; break;
    case at::kFloat: unit = 8; break;
    default: return N;
  }
  const int64_t Np = (N + unit - 1) / unit * unit;
  return N > 0 && Np <= 128 ? Np : N;
}
torch::Tensor pad_columns(const torch::Tensor &t, int64_t Np) {
  if (t.size(2) == Np) return t;
  auto padded = torch::zeros({t.size(0), t.size(1), Np}, t.options());
  padded.narrow(2, 0, t.size(2)).copy_(t);
  return padded;
}
torch::Tensor cut_columns(const torch::Tensor &t, int64_t N) {
  return t.size(2) == N ? t : t.narrow(2, 0, N).contiguous();
}

// Head widths beyond 128 (the widest the tuned kernels take) are worked on in slices of 128 columns:
// results with N columns are independent per slice, bands are the sum over the slices.  The slices
// of a band are computed and summed in float32 whatever the storage type (a 16-bit partial band
// would be rounded at the magnitude of the partial sums, which shows where the slices cancel) and
// the sum is rounded once.  float64 is not sliced: its kernels take every head width.
constexpr int64_t kMaxWidth = 128;
bool sliced_width(const torch::Tensor &t, int64_t w) {
  return t.size(2) > kMaxWidth && !tiles_preferred(t, w) && (t.scalar_type() == at::kHalf || t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat);
}

wm_operand operand(const torch::Tensor &t) {
  return wm_operand{t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)};
}

void raise_on_error(int status, const char *op) {
  TORCH_CHECK(status == WM_OK, op, ": ", wm_status_string(status), " (status ", status, ")");
}

void *current_stream(const torch::Tensor &t) {
  return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// K comes as (B,N,M).  The kernels want key rows contiguous, which is what a
// transposed view of a row-major (B,M,N) tensor already is; anything else is
// copied into that layout once (the reference always copies: cuda:236).
// A tensor that is laid out as (B,N,M) with unit stride along M goes through the library's own
// transpose (one read and one write at memory speed; a general strided copy reaches a quarter of that).
torch::Tensor key_rows(const torch::Tensor &k) {
  auto view = k.transpose(1, 2);
  if (view.stride(2) == 1 || k.stride(2) != 1 || k.numel() == 0 || !k.is_cuda()) return vector_friendly(view);
  const int64_t es = k.element_size();
  if (es != 2 && es != 4 && es != 8) return vector_friendly(view);
  auto rows = torch::empty({k.size(0), k.size(2), k.size(1)}, k.options());
  const wm_operand src{k.data_ptr(), k.stride(0), k.stride(1), k.stride(2)};
  const int dtype = es == 2 ? WM_DTYPE_BF16 : es == 4 ? WM_DTYPE_F32 : WM_DTYPE_F64;  // only the element size matters
  const int status = wm_key_rows(&src, rows.data_ptr(), k.size(0), k.size(1), k.size(2), dtype,
                                 current_stream(k));
  if (status == WM_ERR_UNSUPPORTED) return vector_friendly(view);  // odd alignment: the general copy
  raise_on_error(status, "key rows");
  return rows;
}


void check_window_inputs(const torch::Tensor &src, const torch::Tensor &other) {
  check_gpu(src, "A");
  check_gpu(other, "B");
  TORCH_CHECK(src.dim() == 3 && other.dim() == 3, "Input mismatch");
  TORCH_CHECK(src.size(0) == other.size(0), "Input mismatch");
  TORCH_CHECK(src.size(2) == other.size(1), "Input mismatch");
  TORCH_CHECK(src.size(1) == other.size(2), "Input mismatch");
  TORCH_CHECK(src.scalar_type() == other.scalar_type(), "Input mismatch");
  TORCH_CHECK(src.device() == other.device(), "Input mismatch");
}

void check_unwindow_inputs(const torch::Tensor &src, const torch::Tensor &other, int64_t w) {
  check_gpu(src, "A");
  check_gpu(other, "B");
  TORCH_CHECK(src.dim() == 3 && other.dim() == 3, "Input mismatch");
  TORCH_CHECK(src.size(0) == other.size(0), "Input mismatch");
  TORCH_CHECK(src.size(2) == 2 * w + 1, "Input mismatch");
  TORCH_CHECK(src.size(1) == other.size(1), "Input mismatch");
  TORCH_CHECK(src.scalar_type() == other.scalar_type(), "Input mismatch");
  TORCH_CHECK(src.device() == other.device(), "Input mismatch");
}

void check_grad(const torch::Tensor &g, const torch::Tensor &like, std::vector<int64_t> sizes) {
  check_gpu(g, "grad_C");
  TORCH_CHECK(g.dim() == 3 && g.sizes().vec() == sizes, "Input mismatch");
  TORCH_CHECK(g.scalar_type() == like.scalar_type() && g.device() == like.device(), "Input mismatch");
}

// reference: window_matmul_forward -> window_matmul_fw_cuda (window_matmul.cpp:74-78, cuda:224-270)
torch::Tensor window_matmul_forward(torch::Tensor src, torch::Tensor other, int64_t window_size) {
  TORCH_CHECK(window_size >= 0, "Input mismatch");
  check_window_inputs(src, other);
  const int dtype = abi_dtype(src, "window_matmul_fw_cuda");
  at::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  if (sliced_width(src, window_size)) {
    torch::Tensor band;
    for (int64_t h = 0; h < src.size(2); h += kMaxWidth) {
      const int64_t n = std::min(kMaxWidth, src.size(2) - h);
      auto part = window_matmul_forward(src.narrow(2, h, n).to(at::kFloat), other.narrow(1, h, n).to(at::kFloat), window_size);
      if (h == 0) band = part; else band.add_(part);
    }
    return band.to(src.scalar_type());
  }
  const int64_t B = src.size(0), M = src.size(1), N = padded_width(src, window_size);
  auto q = vector_friendly(pad_columns(src, N));
  auto krows = pad_columns(key_rows(other), N);  // (B,M,N) view or copy
  auto kt = krows.transpose(1, 2);
  auto out = torch::empty({B, M, 2 * window_size + 1}, src.options());
  wm_operand oq = operand(q), ok = operand(kt), oa = operand(out);
  raise_on_error(wm_window_matmul_forward(&oq, &ok, &oa, B, M, N, window_size, dtype, 0, current_stream(src)),
                 "window_matmul_forward");
  return out;
}

// reference: window_matmul_backward -> window_matmul_bw_cuda (window_matmul.cpp:80-85, cuda:272-319)
// need_src / need_other (extensions of the reference signature, both true by default) let the
// autograd Function skip the kernel of a gradient nobody asked for; a skipped one comes back as None.
std::tuple<c10::optional<torch::Tensor>, c10::optional<torch::Tensor>> window_matmul_backward(
    torch::Tensor src, torch::Tensor other, int64_t window_size, torch::Tensor grad_output, bool need_src,
    bool need_other) {
  TORCH_CHECK(window_size >= 0, "Input mismatch");
  check_window_inputs(src, other);
  const int64_t B = src.size(0), M = src.size(1), N = src.size(2);
  check_grad(grad_output, src, {B, M, 2 * window_size + 1});
  const int dtype = abi_dtype(src, "window_matmul_bw_cuda");
  at::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  if (sliced_width(src, window_size)) {
    std::vector<torch::Tensor> gq, gk;
    for (int64_t h = 0; h < N; h += kMaxWidth) {
      const int64_t n = std::min(kMaxWidth, N - h);
      auto part = window_matmul_backward(src.narrow(2, h, n), other.narrow(1, h, n), window_size, grad_output, need_src, need_other);
      if (need_src) gq.push_back(*std::get<0>(part));
      if (need_other) gk.push_back(*std::get<1>(part));
    }
    c10::optional<torch::Tensor> grad_q, grad_k;
    if (need_src) grad_q = torch::cat(gq, 2);
    if (need_other) grad_k = torch::cat(gk, 1);
    return std::make_tuple(grad_q, grad_k);
  }
  const int64_t Np = padded_width(src, window_size);
  auto q = vector_friendly(pad_columns(src, Np));
  auto kt = pad_columns(key_rows(other), Np).transpose(1, 2);
  auto ga = band_friendly(grad_output);
  c10::optional<torch::Tensor> grad_q, grad_k;
  if (need_src) grad_q = torch::empty({B, M, Np}, src.options());
  // grad_k is produced row-major per key row and handed back in the (B,N,M)
  // orientation of `other` as a transposed view, like the reference (cuda:318).
  if (need_other) grad_k = torch::empty({B, M, Np}, src.options()).transpose(1, 2);
  wm_operand oq = operand(q), ok = operand(kt), oga = operand(ga), ogq{}, ogk{};
  if (need_src) ogq = operand(*grad_q);
  if (need_other) ogk = operand(*grad_k);
  raise_on_error(wm_window_matmul_backward(&oq, &ok, &oga, need_src ? &ogq : nullptr, need_other ? &ogk : nullptr, B,
                                           M, Np, window_size, dtype, 0, current_stream(src)),
                 "window_matmul_backward");
  if (need_src) grad_q = cut_columns(*grad_q, N);
  if (need_other && Np != N) grad_k = grad_k->narrow(1, 0, N);
  return std::make_tuple(grad_q, grad_k);
}

// reference: unwindow_matmul_forward -> unwindow_matmul_fw_cuda (window_matmul.cpp:87-91, cuda:321-358)
torch::Tensor unwindow_matmul_forward(torch::Tensor src, torch::Tensor other, int64_t window_size) {
  TORCH_CHECK(window_size >= 0, "Input mismatch");
  check_unwindow_inputs(src, other, window_size);
  const int dtype = abi_dtype(src, "unwindow_matmul_fw_cuda");
  at::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  const int64_t B = other.size(0), M = other.size(1), N = other.size(2);
  if (sliced_width(other, window_size)) {
    std::vector<torch::Tensor> parts;
    for (int64_t h = 0; h < N; h += kMaxWidth)
      parts.push_back(unwindow_matmul_forward(src, other.narrow(2, h, std::min(kMaxWidth, N - h)), window_size));
    return torch::cat(parts, 2);
  }
  const int64_t Np = padded_width(other, window_size);
  auto a = band_friendly(src);
  auto v = vector_friendly(pad_columns(other, Np));
  auto out = torch::empty({B, M, Np}, src.options());
  wm_operand oa = operand(a), ov = operand(v), oo = operand(out);
  raise_on_error(wm_unwindow_matmul_forward(&oa, &ov, &oo, B, M, Np, window_size, dtype, 0, current_stream(src)),
                 "unwindow_matmul_forward");
  return cut_columns(out, N);
}

// reference: unwindow_matmul_backward -> unwindow_matmul_bw_cuda (window_matmul.cpp:93-98, cuda:360-416)
std::tuple<c10::optional<torch::Tensor>, c10::optional<torch::Tensor>> unwindow_matmul_backward(
    torch::Tensor src, torch::Tensor other, int64_t window_size, torch::Tensor grad_output, bool need_src,
    bool need_other) {
  TORCH_CHECK(window_size >= 0, "Input mismatch");
  check_unwindow_inputs(src, other, window_size);
  const int64_t B = other.size(0), M = other.size(1), N = other.size(2);
  check_grad(grad_output, src, {B, M, N});
  const int dtype = abi_dtype(src, "unwindow_matmul_bw_cuda");
  at::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  if (sliced_width(other, window_size)) {
    c10::optional<torch::Tensor> grad_a, grad_v;
    std::vector<torch::Tensor> gv;
    for (int64_t h = 0; h < N; h += kMaxWidth) {
      const int64_t n = std::min(kMaxWidth, N - h);
      if (need_other)
        gv.push_back(*std::get<1>(unwindow_matmul_backward(src, other.narrow(2, h, n), window_size, grad_output.narrow(2, h, n), false, true)));
      if (need_src) {  // grad_a = band of grad_output against other: in float32, as in window_matmul_forward
        auto part = window_matmul_forward(grad_output.narrow(2, h, n).to(at::kFloat), other.narrow(2, h, n).transpose(1, 2).to(at::kFloat), window_size);
        if (h == 0) grad_a = part; else grad_a->add_(part);
      }
    }
    if (need_src) grad_a = grad_a->to(src.scalar_type());
    if (need_other) grad_v = torch::cat(gv, 2);
    return std::make_tuple(grad_a, grad_v);
  }
  const int64_t Np = padded_width(other, window_size);
  auto a = band_friendly(src);
  auto v = vector_friendly(pad_columns(other, Np));
  auto go = vector_friendly(pad_columns(grad_output, Np));
  c10::optional<torch::Tensor> grad_a, grad_v;
  if (need_src) grad_a = torch::empty({B, M, 2 * window_size + 1}, src.options());
  if (need_other) grad_v = torch::empty({B, M, Np}, src.options());
  wm_operand oa = operand(a), ov = operand(v), ogo = operand(go), oga{}, ogv{};
  if (need_src) oga = operand(*grad_a);
  if (need_other) ogv = operand(*grad_v);
  raise_on_error(wm_unwindow_matmul_backward(&oa, &ov, &ogo, need_src ? &oga : nullptr, need_other ? &ogv : nullptr, B,
                                             M, Np, window_size, dtype, 0, current_stream(src)),
                 "unwindow_matmul_backward");
  if (need_other) grad_v = cut_columns(*grad_v, N);
  return std::make_tuple(grad_a, grad_v);
}

// Softmax over the band dimension, the step callers put between the two ops
// (reference tests/test_attention.py:60-61); not part of the reference's native module.
torch::Tensor band_softmax_forward(torch::Tensor src, double scale, bool mask_out_of_range) {
  check_gpu(src, "A");
  TORCH_CHECK(src.dim() == 3 && src.size(2) % 2 == 1, "Input mismatch");
  const int dtype = abi_dtype(src, "band_softmax_forward");
  at::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
  auto a = band_friendly(src);
  auto out = torch::empty_like(a);
  wm_operand oa = operand(a), oo = operand(out);
  raise_on_error(wm_band_softmax_forward(&oa, &oo, a.size(0), a.size(1), a.size(2) / 2, scale, mask_out_of_range,
                                         dtype, 0, current_stream(src)),
                 "band_softmax_forward");
  return out;
}

torch::Tensor band_softmax_backward(torch::Tensor probs, torch::Tensor grad_output, double scale,
                                    bool mask_out_of_range) {
  check_gpu(probs, "P");
  check_gpu(grad_output, "grad_P");
  TORCH_CHECK(probs.dim() == 3 && probs.size(2) % 2 == 1, "Input mismatch");
  TORCH_CHECK(grad_output.sizes() == probs.sizes() && grad_output.scalar_type() == probs.scalar_type() &&
                  grad_output.device() == probs.device(),
              "Input mismatch");
  const int dtype = abi_dtype(probs, "band_softmax_backward");
  at::hip::HIPGuardMasqueradingAsCUDA guard(probs.device());
  auto p = band_friendly(probs);
  auto g = band_friendly(grad_output);
  auto out = torch::empty_like(p);
  wm_operand op = operand(p), og = operand(g), oo = operand(out);
  raise_on_error(wm_band_softmax_backward(&op, &og, &oo, p.size(0), p.size(1), p.size(2) / 2, scale,
                                          mask_out_of_range, dtype, 0, current_stream(probs)),
                 "band_softmax_backward");
  return out;
}

// Fused window attention (no counterpart in the reference's native module): forward returns
// (o, lse); q, k, v are (B, M, N) with k holding key rows.  Raises when the fused kernels do not
// cover the problem; window_attention_supported() lets the caller choose the separate ops first.
bool window_attention_supported(torch::Tensor q, int64_t window_size, double scale) {
  if (q.dim() != 3 || !q.device().is_cuda()) return false;
  int dtype;
  switch (q.scalar_type()) {
    case at::kHalf: dtype = WM_DTYPE_F16; break;
    case at::kBFloat16: dtype = WM_DTYPE_BF16; break;
    default: return false;
  }
  return wm_window_attention_supported(q.size(1), q.size(2), window_size, dtype, scale) != 0;
}

void check_attention_inputs(const torch::Tensor &q, const torch::Tensor &k, const torch::Tensor &v) {
  check_gpu(q, "Q");
  check_gpu(k, "K");
  check_gpu(v, "V");
  TORCH_CHECK(q.dim() == 3 && k.sizes() == q.sizes() && v.sizes() == q.sizes(), "Input mismatch");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "Input mismatch");
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "Input mismatch");
}

std::tuple<torch::Tensor, torch::Tensor> window_attention_forward(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                                                  int64_t window_size, double scale,
                                                                  bool mask_out_of_range) {
  check_attention_inputs(q, k, v);
  const int dtype = abi_dtype(q, "window_attention_forward");
  at::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  const int64_t B = q.size(0), M = q.size(1), N = q.size(2);
  auto qq = vector_friendly(q), kk = vector_friendly(k), vv = vector_friendly(v);
  auto o = torch::empty({B, M, N}, q.options());
  auto lse = torch::empty({B, M}, q.options().dtype(at::kFloat));
  wm_operand oq = operand(qq), ok = operand(kk), ov = operand(vv), oo = operand(o);
  raise_on_error(wm_window_attention_forward(&oq, &ok, &ov, &oo, lse.data_ptr<float>(), B, M, N, window_size, scale,
                                             mask_out_of_range, dtype, 0, current_stream(q)),
                 "window_attention_forward");
  return std::make_tuple(o, lse);
}

std::tuple<c10::optional<torch::Tensor>, c10::optional<torch::Tensor>, c10::optional<torch::Tensor>>
window_attention_backward(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o, torch::Tensor lse,
                          torch::Tensor grad_output, int64_t window_size, double scale, bool need_q, bool need_k,
                          bool need_v) {
  check_attention_inputs(q, k, v);
  check_grad(grad_output, q, q.sizes().vec());
  check_grad(o, q, q.sizes().vec());
  TORCH_CHECK(lse.device() == q.device() && lse.scalar_type() == at::kFloat && lse.dim() == 2 &&
                  lse.size(0) == q.size(0) && lse.size(1) == q.size(1) && lse.is_contiguous(),
              "Input mismatch");
  const int dtype = abi_dtype(q, "window_attention_backward");
  at::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  const int64_t B = q.size(0), M = q.size(1), N = q.size(2);
  auto qq = vector_friendly(q), kk = vector_friendly(k), vv = vector_friendly(v), oo = vector_friendly(o),
       go = vector_friendly(grad_output);
  c10::optional<torch::Tensor> gq, gk, gv;
  wm_operand f{}, g{}, h{};
  if (need_q) gq = torch::empty({B, M, N}, q.options()), f = operand(*gq);
  if (need_k) gk = torch::empty({B, M, N}, q.options()), g = operand(*gk);
  if (need_v) gv = torch::empty({B, M, N}, q.options()), h = operand(*gv);
  auto delta = torch::empty({2, B, M}, lse.options());  // row sums and log2-scaled log-sum-exp
  wm_operand a = operand(qq), b = operand(kk), c = operand(vv), d = operand(oo), e = operand(go);
  raise_on_error(wm_window_attention_backward(&a, &b, &c, &d, lse.data_ptr<float>(), &e, need_q ? &f : nullptr,
                                              need_k ? &g : nullptr, need_v ? &h : nullptr, delta.data_ptr<float>(),
                                              B, M, N, window_size, scale, dtype, 0, current_stream(q)),
                 "window_attention_backward");
  return std::make_tuple(gq, gk, gv);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "MI355X banded matmul kernels behind the window_matmul package";
  // The argument lists and workspace sizes of the C ABI change with WM_ABI_VERSION (version 4 doubled
  // the float workspace of wm_window_attention_backward to 2 B M values): a library of another
  // version next to this module would be called with the wrong contract, so refuse to load.
  if (wm_abi_version() != WM_ABI_VERSION)
    throw std::runtime_error("window_matmul_kernel was built against ABI " + std::to_string(WM_ABI_VERSION) +
                             " of libwindow_matmul_hip.so, the library that was loaded reports " +
                             std::to_string(wm_abi_version()));
  m.def("window_matmul_forward", &window_matmul_forward, "WindowMatmul forward");
  m.def("window_matmul_backward", &window_matmul_backward, "WindowMatmul backward", py::arg("src"), py::arg("other"),
        py::arg("window_size"), py::arg("grad_output"), py::arg("need_src") = true, py::arg("need_other") = true);
  m.def("unwindow_matmul_forward", &unwindow_matmul_forward, "UnwindowMatmul forward");
  m.def("unwindow_matmul_backward", &unwindow_matmul_backward, "UnwindowMatmul backward", py::arg("src"),
        py::arg("other"), py::arg("window_size"), py::arg("grad_output"), py::arg("need_src") = true,
        py::arg("need_other") = true);
  m.def("band_softmax_forward", &band_softmax_forward, "softmax over the band dimension", py::arg("src"),
        py::arg("scale") = 1.0, py::arg("mask_out_of_range") = false);
  m.def("band_softmax_backward", &band_softmax_backward, "backward of band_softmax_forward", py::arg("probs"),
        py::arg("grad_output"), py::arg("scale") = 1.0, py::arg("mask_out_of_range") = false);
  m.def("window_attention_supported", &window_attention_supported, "whether the fused attention kernels cover q",
        py::arg("q"), py::arg("window_size"), py::arg("scale"));
  m.def("window_attention_forward", &window_attention_forward, "fused window attention forward -> (o, lse)",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("window_size"), py::arg("scale"),
        py::arg("mask_out_of_range") = false);
  m.def("window_attention_backward", &window_attention_backward, "fused window attention backward -> (gq, gk, gv)",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("o"), py::arg("lse"), py::arg("grad_output"),
        py::arg("window_size"), py::arg("scale"), py::arg("need_q") = true, py::arg("need_k") = true,
        py::arg("need_v") = true);
  m.def("abi_version", []() { return wm_abi_version(); }, "ABI version of libwindow_matmul_hip.so");
}
