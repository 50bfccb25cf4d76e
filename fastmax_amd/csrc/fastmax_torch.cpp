// PyTorch-ROCm binding of the Fastmax C ABI.  The module is named `fastmax_cuda` and exports
// `forwardpass` / `backwardpass` with the positional signatures of the reference extension
// (fastmax_cuda.cpp:17-37).  forwardpass exists in both forms the reference's files call: the
// 13-argument one of the live kernels (fastmax_cuda_forward.cu:297-314; example.py:36,
// model.py:37) and the 14-argument one with rpe_matrix after drop_noise (fastmax_cuda.cpp:17,
// test_fastmax.py:32), so the reference's autograd Functions run on it unchanged.
// `forward_ex` / `backward_ex` are the non-mutating entry points the package's own autograd
// Function uses: they differentiate through the normalisation and accept bf16.
//
// Host code only: tensors, the current stream and the device guard come from torch; all device
// work happens behind include/fastmax_amd.h.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <vector>

#include "fastmax_amd.h"

namespace {

#define CHECK_GPU(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
  CHECK_GPU(x);        \
  CHECK_CONTIGUOUS(x)

void raise_on(int rc) { TORCH_CHECK(rc == FASTMAX_OK, "fastmax: ", fastmax_last_error(), " (code ", rc, ")"); }

fastmax_desc make_desc(const torch::Tensor& q, const torch::Tensor& k, bool mask, bool normalize,
                       double temperature, double a0, double a1, double a2, double lim, int64_t p) {
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3, "q, k, v must be (b*h, n, d)");
  TORCH_CHECK(k.size(2) == q.size(2), "k has head dimension ", k.size(2), " but q has ", q.size(2));
  TORCH_CHECK(q.scalar_type() == torch::kFloat32 || q.scalar_type() == torch::kBFloat16,
              "q must be float32 or bfloat16");
  fastmax_desc ds;
  ds.bh = (int32_t)q.size(0);
  ds.bhkv = (int32_t)k.size(0);
  ds.nq = (int32_t)q.size(1);
  ds.nk = (int32_t)k.size(1);
  ds.d = (int32_t)q.size(2);
  ds.dtype = q.scalar_type() == torch::kFloat32 ? FASTMAX_F32 : FASTMAX_BF16;
  ds.mask = mask;
  ds.normalize = normalize;
  ds.p = (int32_t)p;
  ds.lim = (float)lim;
  ds.temperature = (float)temperature;
  ds.a0 = (float)a0;
  ds.a1 = (float)a1;
  ds.a2 = (float)a2;
  raise_on(fastmax_check_desc(&ds));
  return ds;
}

void check_same(const torch::Tensor& a, const torch::Tensor& b, const char* what) {
  TORCH_CHECK(a.scalar_type() == b.scalar_type() && a.device() == b.device(), what,
              " must share dtype and device with q");
}

torch::Tensor workspace(const fastmax_desc& ds, int pass, const torch::Tensor& like, size_t* bytes) {
  *bytes = fastmax_workspace_bytes(&ds, pass);
  TORCH_CHECK(*bytes > 0, "fastmax: ", fastmax_last_error());
  return torch::empty({(int64_t)*bytes}, like.options().dtype(torch::kUInt8));
}

fastmax_stream_t current_stream(const torch::Tensor& t) {
  return reinterpret_cast<fastmax_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream());
}

// (o, den, qk_scale, qk_argmax, saved_states); o is (bh, n, d).  save_states keeps the prefix
// states for backward_ex (a uint8 tensor; empty when not asked for)
std::vector<torch::Tensor> forward_ex(torch::Tensor q, torch::Tensor k, torch::Tensor v, bool mask,
                                      bool normalize, double temperature, double a0, double a1,
                                      double a2, double lim, int64_t p, bool save_states) {
  CHECK_INPUT(q);
  CHECK_INPUT(k);
  CHECK_INPUT(v);
  check_same(q, k, "k");
  check_same(q, v, "v");
  TORCH_CHECK(k.sizes() == v.sizes(), "k and v must have the same shape");
  const fastmax_desc ds = make_desc(q, k, mask, normalize, temperature, a0, a1, a2, lim, p);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  auto o = torch::empty_like(q);
  auto den = torch::empty({q.size(0), q.size(1)}, q.options().dtype(torch::kFloat32));
  auto scale = torch::empty({2 * q.size(0)}, q.options().dtype(torch::kFloat32));
  auto arg = torch::empty({2 * q.size(0)}, q.options().dtype(torch::kInt32));
  size_t wsb = 0;
  torch::Tensor ws, saved;
  if (save_states) {
    const size_t sb = fastmax_saved_state_bytes(&ds);
    TORCH_CHECK(sb > 0, "fastmax: ", fastmax_last_error());
    saved = torch::empty({(int64_t)sb}, q.options().dtype(torch::kUInt8));
    // the per-head scalars only: the states go to `saved` -- unless the kernels keep nothing (the 256-byte token)
    // and work as in a plain forward pass
    wsb = sb > 256 ? (size_t)16 * ds.bh + 512 : fastmax_workspace_bytes(&ds, FASTMAX_PASS_FORWARD);
    ws = torch::empty({(int64_t)wsb}, q.options().dtype(torch::kUInt8));
  } else {
    saved = torch::empty({0}, q.options().dtype(torch::kUInt8));
    ws = workspace(ds, FASTMAX_PASS_FORWARD, q, &wsb);
  }
  raise_on(fastmax_forward_saving(&ds, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ds.d,
                                  den.data_ptr<float>(), 1, scale.data_ptr<float>(), arg.data_ptr<int32_t>(),
                                  ws.data_ptr(), wsb, save_states ? saved.data_ptr() : nullptr,
                                  (size_t)saved.numel(), current_stream(q)));
  return {o, den, scale, arg, saved};
}

std::vector<torch::Tensor> backward_ex(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                       torch::Tensor o, torch::Tensor den, torch::Tensor go,
                                       torch::Tensor scale, torch::Tensor arg, bool mask,
                                       bool normalize, double temperature, double a0, double a1,
                                       double a2, double lim, int64_t p, torch::Tensor saved) {
  CHECK_INPUT(q);
  CHECK_INPUT(k);
  CHECK_INPUT(v);
  CHECK_INPUT(o);
  CHECK_INPUT(den);
  CHECK_INPUT(go);
  CHECK_INPUT(scale);
  CHECK_INPUT(arg);
  check_same(q, k, "k");
  check_same(q, v, "v");
  check_same(q, o, "o");
  check_same(q, go, "grad_output");
  TORCH_CHECK(k.sizes() == v.sizes(), "k and v must have the same shape");
  TORCH_CHECK(o.sizes() == q.sizes() && go.sizes() == q.sizes(), "o and grad_output must be shaped like q");
  TORCH_CHECK(den.scalar_type() == torch::kFloat32 && den.numel() == q.size(0) * q.size(1), "den must be float32 (bh, n)");
  TORCH_CHECK(scale.scalar_type() == torch::kFloat32 && scale.numel() == 2 * q.size(0), "qk_scale must be float32 (2*bh)");
  TORCH_CHECK(arg.scalar_type() == torch::kInt32 && arg.numel() == 2 * q.size(0), "qk_argmax must be int32 (2*bh)");
  const fastmax_desc ds = make_desc(q, k, mask, normalize, temperature, a0, a1, a2, lim, p);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  auto dq = torch::empty_like(q);
  auto dk = torch::empty_like(k);
  auto dv = torch::empty_like(v);
  size_t wsb = 0;
  auto ws = workspace(ds, FASTMAX_PASS_BACKWARD, q, &wsb);
  const bool have_saved = saved.defined() && saved.numel() > 0;
  if (have_saved) {
    TORCH_CHECK(saved.is_cuda() && saved.is_contiguous() && saved.device() == q.device(),
                "saved_states must be a contiguous tensor on q's device");
  }
  raise_on(fastmax_backward_saved(&ds, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ds.d,
                                  den.data_ptr<float>(), 1, go.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                  dv.data_ptr(), scale.data_ptr<float>(), arg.data_ptr<int32_t>(),
                                  ws.data_ptr(), wsb, have_saved ? saved.data_ptr() : nullptr,
                                  have_saved ? (size_t)(saved.numel() * saved.element_size()) : 0,
                                  current_stream(q)));
  return {dq, dk, dv};
}

// ---- strided tensors -----------------------------------------------------------------------
// q, o, grad_output, dq: (B, G, R, T, D) views (G key/value groups of R query heads); k, v, dk, dv:
// (B, G, T, D) views; any strides with unit channel stride, e.g. slices of the fused projection of a
// GPT block (model.py:474-499) -- no .contiguous() copies (model.py:572-574) and no transpose of the
// result (model.py:603).
fastmax_strides strides5(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 5 && t.stride(4) == 1, name, " must be a (B, G, R, T, D) view with unit channel stride");
  return fastmax_strides{t.stride(0), t.stride(1), t.stride(2), t.stride(3)};
}
fastmax_strides strides4(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 4 && t.stride(3) == 1, name, " must be a (B, G, T, D) view with unit channel stride");
  return fastmax_strides{t.stride(0), t.stride(1), 0, t.stride(2)};
}
fastmax_desc make_desc5(const torch::Tensor& q, const torch::Tensor& k, bool mask, bool normalize,
                        double temperature, double a0, double a1, double a2, double lim, int64_t p) {
  TORCH_CHECK(q.dim() == 5 && k.dim() == 4 && k.size(0) == q.size(0) && k.size(1) == q.size(1) && k.size(3) == q.size(4),
              "q must be (B, G, R, T, D) and k, v (B, G, T, D)");
  TORCH_CHECK(q.scalar_type() == torch::kFloat32 || q.scalar_type() == torch::kBFloat16, "q must be float32 or bfloat16");
  fastmax_desc ds;
  ds.bh = (int32_t)(q.size(0) * q.size(1) * q.size(2));
  ds.bhkv = (int32_t)(q.size(0) * q.size(1));
  ds.nq = (int32_t)q.size(3);
  ds.nk = (int32_t)k.size(2);
  ds.d = (int32_t)q.size(4);
  ds.dtype = q.scalar_type() == torch::kFloat32 ? FASTMAX_F32 : FASTMAX_BF16;
  ds.mask = mask;
  ds.normalize = normalize;
  ds.p = (int32_t)p;
  ds.lim = (float)lim;
  ds.temperature = (float)temperature;
  ds.a0 = (float)a0;
  ds.a1 = (float)a1;
  ds.a2 = (float)a2;
  raise_on(fastmax_check_desc(&ds));
  return ds;
}

// (o, den, qk_scale, qk_argmax, saved_states); o is the (B, G, R, T, D) view of freshly allocated
// token-major (B, T, G, R, D) memory.
std::vector<torch::Tensor> forward_strided(torch::Tensor q, torch::Tensor k, torch::Tensor v, bool mask,
                                           bool normalize, double temperature, double a0, double a1,
                                           double a2, double lim, int64_t p, bool save_states) {
  CHECK_GPU(q);
  CHECK_GPU(k);
  CHECK_GPU(v);
  check_same(q, k, "k");
  check_same(q, v, "v");
  TORCH_CHECK(k.sizes() == v.sizes(), "k and v must have the same shape");
  const fastmax_desc ds = make_desc5(q, k, mask, normalize, temperature, a0, a1, a2, lim, p);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  auto o = torch::empty({q.size(0), q.size(3), q.size(1), q.size(2), q.size(4)}, q.options()).permute({0, 2, 3, 1, 4});
  fastmax_layout lay{};
  lay.groups = (int32_t)q.size(1);
  lay.q = strides5(q, "q");
  lay.k = strides4(k, "k");
  lay.v = strides4(v, "v");
  lay.o = strides5(o, "o");
  auto den = torch::empty({(int64_t)ds.bh, q.size(3)}, q.options().dtype(torch::kFloat32));
  auto scale = torch::empty({2 * (int64_t)ds.bh}, q.options().dtype(torch::kFloat32));
  auto arg = torch::empty({2 * (int64_t)ds.bh}, q.options().dtype(torch::kInt32));
  size_t wsb = 0;
  torch::Tensor ws, saved;
  if (save_states) {
    const size_t sb = fastmax_saved_state_bytes_strided(&ds, &lay);
    TORCH_CHECK(sb > 0, "fastmax: ", fastmax_last_error());
    saved = torch::empty({(int64_t)sb}, q.options().dtype(torch::kUInt8));
    wsb = sb > 256 ? (size_t)16 * ds.bh + 512 : fastmax_workspace_bytes_strided(&ds, &lay, FASTMAX_PASS_FORWARD);   // (as in forward_ex)
  } else {
    saved = torch::empty({0}, q.options().dtype(torch::kUInt8));
    wsb = fastmax_workspace_bytes_strided(&ds, &lay, FASTMAX_PASS_FORWARD);
    TORCH_CHECK(wsb > 0, "fastmax: ", fastmax_last_error());
  }
  ws = torch::empty({(int64_t)wsb}, q.options().dtype(torch::kUInt8));
  raise_on(fastmax_forward_strided(&ds, &lay, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                   den.data_ptr<float>(), 1, scale.data_ptr<float>(), arg.data_ptr<int32_t>(),
                                   ws.data_ptr(), wsb, save_states ? saved.data_ptr() : nullptr,
                                   (size_t)saved.numel(), current_stream(q)));
  return {o, den, scale, arg, saved};
}

// Writes dq, dk, dv into the views the caller hands in (e.g. slices of the gradient of the fused
// projection).
void backward_strided(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor o, torch::Tensor den,
                      torch::Tensor go, torch::Tensor scale, torch::Tensor arg, torch::Tensor dq, torch::Tensor dk,
                      torch::Tensor dv, bool mask, bool normalize, double temperature, double a0, double a1,
                      double a2, double lim, int64_t p, torch::Tensor saved) {
  for (const torch::Tensor* t : {&q, &k, &v, &o, &go, &dq, &dk, &dv}) {
    TORCH_CHECK(t->device().is_cuda() && t->device() == q.device() && t->scalar_type() == q.scalar_type(),
                "all tensors must live on q's device and share its dtype");
  }
  CHECK_INPUT(den);
  CHECK_INPUT(scale);
  CHECK_INPUT(arg);
  TORCH_CHECK(o.sizes() == q.sizes() && go.sizes() == q.sizes() && dq.sizes() == q.sizes(), "o, grad_output and dq must be shaped like q");
  TORCH_CHECK(k.sizes() == v.sizes() && dk.sizes() == k.sizes() && dv.sizes() == k.sizes(), "v, dk and dv must be shaped like k");
  const fastmax_desc ds = make_desc5(q, k, mask, normalize, temperature, a0, a1, a2, lim, p);
  TORCH_CHECK(den.scalar_type() == torch::kFloat32 && den.numel() == (int64_t)ds.bh * ds.nq, "den must be float32 (bh, n)");
  TORCH_CHECK(scale.scalar_type() == torch::kFloat32 && scale.numel() == 2 * (int64_t)ds.bh, "qk_scale must be float32 (2*bh)");
  TORCH_CHECK(arg.scalar_type() == torch::kInt32 && arg.numel() == 2 * (int64_t)ds.bh, "qk_argmax must be int32 (2*bh)");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  fastmax_layout lay{};
  lay.groups = (int32_t)q.size(1);
  lay.q = strides5(q, "q");
  lay.k = strides4(k, "k");
  lay.v = strides4(v, "v");
  lay.o = strides5(o, "o");
  lay.go = strides5(go, "grad_output");
  lay.dq = strides5(dq, "dq");
  lay.dk = strides4(dk, "dk");
  lay.dv = strides4(dv, "dv");
  const size_t wsb = fastmax_workspace_bytes_strided(&ds, &lay, FASTMAX_PASS_BACKWARD);
  TORCH_CHECK(wsb > 0, "fastmax: ", fastmax_last_error());
  auto ws = torch::empty({(int64_t)wsb}, q.options().dtype(torch::kUInt8));
  const bool have_saved = saved.defined() && saved.numel() > 0;
  raise_on(fastmax_backward_strided(&ds, &lay, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                    den.data_ptr<float>(), 1, go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                    scale.data_ptr<float>(), arg.data_ptr<int32_t>(), ws.data_ptr(), wsb,
                                    have_saved ? saved.data_ptr() : nullptr,
                                    have_saved ? (size_t)(saved.numel() * saved.element_size()) : 0, current_stream(q)));
}

// Reference signature and side effects (fastmax_cuda.cpp:17-24, fastmax_cuda_forward.cu:366-399):
// k is divided by temperature and q, k are normalised IN PLACE, so that the caller's saved
// q, k are the ones backwardpass expects; the result is (bh, nq, d+1) with the row denominators
// in column d; dropout > 0 multiplies the output by 1 + dropout * drop_noise.
// k, v longer than q (fastmax_cuda_forward.cu:109-150: the first nk - nq keys are visible to
// every query) go to the library as they are: the descriptor carries nq and nk.
torch::Tensor forwardpass(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor drop_noise,
                          bool mask, double dropout, bool normalize, double temperature, double a0,
                          double a1, double a2, double lim, int64_t p) {
  CHECK_INPUT(q);
  CHECK_INPUT(k);
  CHECK_INPUT(v);
  check_same(q, k, "k");
  check_same(q, v, "v");
  TORCH_CHECK(q.scalar_type() == torch::kFloat32, "forwardpass takes float32 tensors (use forward_ex for bfloat16)");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3, "q, k, v must be (b*h, n, d)");
  TORCH_CHECK(k.sizes() == v.sizes() && k.size(2) == q.size(2),
              "k and v must have the same shape and q's head dimension");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  fastmax_desc ds = make_desc(q, k, mask, normalize, 1.0, a0, a1, a2, lim, p);
  const fastmax_stream_t stream = current_stream(q);
  if (temperature != 1.0) k.div_(temperature);
  if (normalize) {
    auto nws = torch::empty({16 * (int64_t)ds.bh + 1024}, q.options().dtype(torch::kUInt8));
    raise_on(fastmax_normalize_inplace(&ds, q.data_ptr(), k.data_ptr(), nws.data_ptr(), (size_t)nws.numel(), stream));
    ds.normalize = 0;
  }
  const int64_t d = q.size(2);
  auto o = torch::empty({q.size(0), q.size(1), d + 1}, q.options());
  size_t wsb = 0;
  auto ws = workspace(ds, FASTMAX_PASS_FORWARD, q, &wsb);
  raise_on(fastmax_forward(&ds, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d + 1,
                           o.data_ptr<float>() + d, d + 1, nullptr, nullptr, ws.data_ptr(), wsb, stream));
  if (dropout > 0.0) {
    TORCH_CHECK(drop_noise.defined() && drop_noise.sizes() == q.sizes(), "drop_noise must be shaped like q");
    o.narrow(2, 0, d).mul_(drop_noise * dropout + 1.0);
  }
  return o;
}

// Reference signature (fastmax_cuda.cpp:26-32): q, k as left by forwardpass (already scaled),
// o with the denominator column; no gradient flows through the normalisation here, exactly
// like the reference kernels (fastmax_cuda_backward.cu:900-1006).  grad_output is not modified.
std::vector<torch::Tensor> backwardpass(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                                        torch::Tensor o, torch::Tensor grad_output, bool mask,
                                        double a0, double a1, double a2, int64_t p) {
  CHECK_INPUT(q);
  CHECK_INPUT(k);
  CHECK_INPUT(v);
  CHECK_INPUT(o);
  CHECK_INPUT(grad_output);
  check_same(q, k, "k");
  check_same(q, v, "v");
  check_same(q, o, "o");
  check_same(q, grad_output, "grad_output");
  TORCH_CHECK(q.scalar_type() == torch::kFloat32, "backwardpass takes float32 tensors (use backward_ex for bfloat16)");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3, "q, k, v must be (b*h, n, d)");
  const int64_t d = q.size(2);
  TORCH_CHECK(o.dim() == 3 && o.size(0) == q.size(0) && o.size(1) == q.size(1) && o.size(2) == d + 1,
              "o must be the (bh, n, d+1) tensor forwardpass returned");
  TORCH_CHECK(grad_output.sizes() == q.sizes(), "grad_output must be shaped like q");
  TORCH_CHECK(k.sizes() == v.sizes() && k.size(2) == d, "k and v must have the same shape and q's head dimension");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  const fastmax_desc ds = make_desc(q, k, mask, false, 1.0, a0, a1, a2, 1.0, p);
  auto dq = torch::empty_like(q);
  auto dk = torch::empty_like(k);
  auto dv = torch::empty_like(v);
  size_t wsb = 0;
  auto ws = workspace(ds, FASTMAX_PASS_BACKWARD, q, &wsb);
  raise_on(fastmax_backward(&ds, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d + 1,
                            o.data_ptr<float>() + d, d + 1, grad_output.data_ptr(), dq.data_ptr(),
                            dk.data_ptr(), dv.data_ptr(), nullptr, nullptr, ws.data_ptr(), wsb,
                            current_stream(q)));
  return {dq, dk, dv};
}

// The 14-argument form (fastmax_cuda.cpp:17, called at test_fastmax.py:32): rpe_matrix sits between
// drop_noise and mask.  The relative positional encoding is switched off in every kernel of the
// reference (README.md:16), so the matrix is accepted and not read.
torch::Tensor forwardpass_rpe(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor drop_noise,
                              torch::Tensor rpe_matrix, bool mask, double dropout, bool normalize,
                              double temperature, double a0, double a1, double a2, double lim, int64_t p) {
  (void)rpe_matrix;
  return forwardpass(q, k, v, drop_noise, mask, dropout, normalize, temperature, a0, a1, a2, lim, p);
}

// Bytes of the buffer forward_ex(save_states = true) would allocate for these tensors.
int64_t saved_state_bytes(torch::Tensor q, torch::Tensor k, bool mask, int64_t p) {
  const fastmax_desc ds = make_desc(q, k, mask, false, 1.0, 1.0, 1.0, 0.5, 1.0, p);
  const size_t sb = fastmax_saved_state_bytes(&ds);
  TORCH_CHECK(sb > 0, "fastmax: ", fastmax_last_error());
  return (int64_t)sb;
}

int64_t saved_state_bytes_strided(torch::Tensor q, torch::Tensor k, bool mask, int64_t p) {
  const fastmax_desc ds = make_desc5(q, k, mask, false, 1.0, 1.0, 1.0, 0.5, 1.0, p);
  fastmax_layout lay{};
  lay.groups = (int32_t)q.size(1);
  lay.q = strides5(q, "q");
  lay.k = lay.v = strides4(k, "k");
  // the output forward_strided writes: token-major (B, T, G, R, D) memory seen as (B, G, R, T, D)
  const int64_t G = q.size(1), R = q.size(2), T = q.size(3), D = q.size(4);
  lay.o = fastmax_strides{T * G * R * D, R * D, D, G * R * D};
  const size_t sb = fastmax_saved_state_bytes_strided(&ds, &lay);
  TORCH_CHECK(sb > 0, "fastmax: ", fastmax_last_error());
  return (int64_t)sb;
}

}  // namespace

PYBIND11_MODULE(fastmax_cuda, m) {
  m.def("forwardpass", &forwardpass, "forwardpass");
  m.def("forwardpass", &forwardpass_rpe, "forwardpass with rpe_matrix (accepted, not used)");
  m.def("saved_state_bytes", &saved_state_bytes, "size of the prefix states forward_ex can keep");
  m.def("backwardpass", &backwardpass, "backwardpass");
  m.def("forward_ex", &forward_ex, "forward returning (o, den, qk_scale, qk_argmax, saved_states)");
  m.def("backward_ex", &backward_ex, "backward through the normalisation, returns [dq, dk, dv]");
  m.def("saved_state_bytes_strided", &saved_state_bytes_strided, "the same for strided (B, G, R, T, D) / (B, G, T, D) views");
  m.def("forward_strided", &forward_strided, "forward on strided (B, G, R, T, D) / (B, G, T, D) views");
  m.def("backward_strided", &backward_strided, "backward on strided views, writes dq, dk, dv in place");
  m.def("version", []() { return std::string(fastmax_version()); });
}
