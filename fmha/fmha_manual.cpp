// Host side of the `mha_manual` PyTorch extension for ROCm.
//
// Registers the operators of the reference under the same names and argument
// orders (reference fmha/fmha_manual.cpp:1218-1250):
//   torch.ops.mha_manual.fmha_nvfuser(input, qk, v, amask)                          -> Tensor
//   torch.ops.mha_manual.fmha_train_nvfuser(input, qk, v, pad_mask, dropout_mask)   -> Tensor
//   torch.ops.mha_manual.fmha_train_saveim_nvfuser(same five)                       -> Tensor[]
// and, beyond the reference, the general forward / backward pair
//   torch.ops.mha_manual.fmha_fwd / fmha_bwd / fmha_philox_keep_mask.
//
// There is no fusion compiler here and no device code: this file validates the
// tensors, allocates the outputs, picks up torch's current HIP stream and calls the
// C ABI of libfmha_hip.so (include/fmha_capi.h), which holds the hand-written gfx950
// kernels.  The lazy compile-and-cache runner of the reference
// (common/manual_scheduled_kernel.h:13-41) has no counterpart: nothing is compiled
// at run time, so the ops are stateless and re-entrant.
#include <ATen/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <cmath>
#include <tuple>
#include <vector>

#include "include/fmha_capi.h"

namespace {

struct MaskLayout {
  at::Tensor t; // keeps the (possibly reshaped) mask alive
  int64_t bh_div = 1, stride_b = 0, stride_q = 0;
};

void *current_stream(const at::Tensor &t) {
  return static_cast<void *>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

int dtype_code(const at::Tensor &t) {
  if (t.scalar_type() == at::kHalf) return FMHA_DTYPE_F16;
  if (t.scalar_type() == at::kBFloat16) return FMHA_DTYPE_BF16;
  TORCH_CHECK(false, "mha_manual: tensors must be float16 or bfloat16, got ", t.scalar_type());
  return -1;
}

void check_qkv(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v) {
  TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), "mha_manual: q/k/v must live on the GPU");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, "mha_manual: q/k/v must be [B*H, S, D]");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(),
              "mha_manual: q/k/v must share one dtype");
  TORCH_CHECK(k.size(0) == q.size(0) && v.size(0) == q.size(0) && k.size(2) == q.size(2) &&
                  v.size(2) == q.size(2) && v.size(1) == k.size(1),
              "mha_manual: shapes must be q [BH,Sq,D], k [BH,Sk,D], v [BH,Sk,D]");
  TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && v.is_contiguous(),
              "mha_manual: q/k/v must be contiguous");
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "mha_manual: q/k/v on different devices");
}

// Accepts [BH,Sq,Sk], [BH,1,Sk], [B,1,1,Sk] or [B,1,Sq,Sk] (B dividing BH).
MaskLayout mask_layout(const at::Tensor &mask_in, const at::Tensor &q, int64_t sk, const char *what) {
  const int64_t bh = q.size(0), sq = q.size(1);
  TORCH_CHECK(mask_in.is_cuda() && mask_in.device() == q.device(), "mha_manual: ", what, " must be on q's device");
  TORCH_CHECK(mask_in.scalar_type() == q.scalar_type(), "mha_manual: ", what, " must have q's dtype");
  at::Tensor m = mask_in;
  if (m.dim() == 4) {
    TORCH_CHECK(m.size(1) == 1, "mha_manual: 4-d ", what, " must be [B,1,Sq|1,Sk]");
    m = m.reshape({m.size(0), m.size(2), m.size(3)});
  }
  TORCH_CHECK(m.dim() == 3 && m.size(2) == sk && (m.size(1) == 1 || m.size(1) == sq) && m.size(0) >= 1 &&
                  bh % m.size(0) == 0,
              "mha_manual: ", what, " of shape ", mask_in.sizes(), " does not broadcast over [", bh, ",", sq, ",",
              sk, "]");
  MaskLayout L;
  L.t = m.contiguous();
  L.bh_div = bh / m.size(0);
  L.stride_b = m.size(1) * sk;
  L.stride_q = m.size(1) == 1 ? 0 : sk;
  return L;
}

void fill_common(fmha_fwd_params &p, const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                 const at::Tensor &o, double scale) {
  p.q = q.data_ptr();
  p.k = k.data_ptr();
  p.v = v.data_ptr();
  p.o = o.data_ptr();
  p.bh = static_cast<int32_t>(q.size(0));
  p.sq = static_cast<int32_t>(q.size(1));
  p.sk = static_cast<int32_t>(k.size(1));
  p.d = static_cast<int32_t>(q.size(2));
  p.dtype = dtype_code(q);
  p.scale = static_cast<float>(scale);
}

void launch_fwd(const fmha_fwd_params &p, const at::Tensor &q) {
  const int rc = fmha_fwd_launch(&p, current_stream(q));
  TORCH_CHECK(rc == FMHA_OK, "mha_manual forward: ", fmha_strerror(rc));
}

double default_scale(const at::Tensor &q) { return 1.0 / std::sqrt(static_cast<double>(q.size(2))); }

} // namespace

// ---- the reference's three operators -------------------------------------------------

// Inference forward; `amask` holds 1 where a key is visible and 0 where it is not and
// enters the scores as (1 - amask) * -10000 (reference fmha/fmha_manual.cpp:64-71).
at::Tensor fmha_nvfuser(const at::Tensor &input, const at::Tensor &qk, const at::Tensor &v,
                        const at::Tensor &amask) {
  check_qkv(input, qk, v);
  at::DeviceGuard guard(input.device());
  MaskLayout m = mask_layout(amask, input, qk.size(1), "amask");
  at::Tensor o = at::empty_like(input);
  fmha_fwd_params p = {};
  fill_common(p, input, qk, v, o, default_scale(input));
  p.mask = m.t.data_ptr();
  p.mask_kind = FMHA_MASK_KEEP01;
  p.mask_neg = -10000.f;
  p.mask_bh_div = m.bh_div;
  p.mask_stride_b = m.stride_b;
  p.mask_stride_q = m.stride_q;
  launch_fwd(p, input);
  return o;
}

namespace {

// Train forward with caller-made masks: additive `pad_mask`, multiplicative
// `dropout_mask` whose kept entries are scaled by 1/0.5 (reference
// fmha/fmha_manual.cpp:421,463,478-480; the constant is the keep probability there).
std::vector<at::Tensor> train_forward(const at::Tensor &input, const at::Tensor &qk, const at::Tensor &v,
                                      const at::Tensor &pad_mask, const at::Tensor &dropout_mask, bool save) {
  check_qkv(input, qk, v);
  at::DeviceGuard guard(input.device());
  const int64_t bh = input.size(0), sq = input.size(1), sk = qk.size(1);
  MaskLayout m = mask_layout(pad_mask, input, sk, "pad_mask");
  TORCH_CHECK(dropout_mask.is_cuda() && dropout_mask.device() == input.device() &&
                  dropout_mask.scalar_type() == input.scalar_type() && dropout_mask.dim() == 3 &&
                  dropout_mask.size(0) == bh && dropout_mask.size(1) == sq && dropout_mask.size(2) == sk,
              "mha_manual: dropout_mask must be a [BH,Sq,Sk] tensor of q's dtype on q's device");
  at::Tensor dm = dropout_mask.contiguous();
  at::Tensor o = at::empty_like(input);
  fmha_fwd_params p = {};
  fill_common(p, input, qk, v, o, default_scale(input));
  p.mask = m.t.data_ptr();
  p.mask_kind = FMHA_MASK_ADDITIVE;
  p.mask_bh_div = m.bh_div;
  p.mask_stride_b = m.stride_b;
  p.mask_stride_q = m.stride_q;
  p.drop_kind = FMHA_DROP_TENSOR;
  p.drop_mask = dm.data_ptr();
  p.drop_scale = 2.0f;
  std::vector<at::Tensor> out{o};
  if (save) {
    at::Tensor sm = at::empty({bh, sq, sk}, input.options());
    at::Tensor dr = at::empty({bh, sq, sk}, input.options());
    p.save_softmax = sm.data_ptr();
    p.save_dropout = dr.data_ptr();
    out.push_back(sm);
    out.push_back(dr);
  }
  launch_fwd(p, input);
  return out;
}

} // namespace

at::Tensor fmha_train_nvfuser(const at::Tensor &input, const at::Tensor &qk, const at::Tensor &v,
                              const at::Tensor &pad_mask, const at::Tensor &dropout_mask) {
  return train_forward(input, qk, v, pad_mask, dropout_mask, false)[0];
}

// Returns {context, softmax, dropout_out} in that order (reference fmha/fmha_manual.cpp:894-897).
std::vector<at::Tensor> fmha_train_saveim_nvfuser(const at::Tensor &input, const at::Tensor &qk,
                                                  const at::Tensor &v, const at::Tensor &pad_mask,
                                                  const at::Tensor &dropout_mask) {
  return train_forward(input, qk, v, pad_mask, dropout_mask, true);
}

// ---- general forward / backward (not in the reference) -------------------------------

// Optional valid key counts: an int32 vector of B entries on q's device, B dividing BH.
template <typename P> void set_kv_len(P &p, const c10::optional<at::Tensor> &kv_len, const at::Tensor &q,
                                      at::Tensor &keep) {
  if (!kv_len.has_value() || !kv_len->defined()) return;
  TORCH_CHECK(kv_len->is_cuda() && kv_len->scalar_type() == at::kInt && kv_len->dim() == 1 && kv_len->numel() > 0 &&
                  q.size(0) % kv_len->numel() == 0,
              "mha_manual: kv_len must be an int32 GPU vector whose length divides BH");
  keep = kv_len->contiguous();
  p.kv_len = keep.data_ptr<int32_t>();
  p.kv_len_bh_div = static_cast<int32_t>(q.size(0) / keep.numel());
}

// scale <= 0 selects 1/sqrt(D).  Dropout decisions come from Philox4x32-10 keyed by
// (seed, offset); p_drop == 0 disables dropout.  Returns (O, LSE[bh,sq] fp32).
std::tuple<at::Tensor, at::Tensor> fmha_fwd(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                                            const c10::optional<at::Tensor> &mask, double scale, bool is_causal,
                                            double p_drop, int64_t seed, int64_t offset,
                                            const c10::optional<at::Tensor> &kv_len) {
  check_qkv(q, k, v);
  at::DeviceGuard guard(q.device());
  at::Tensor o = at::empty_like(q);
  at::Tensor lse = at::empty({q.size(0), q.size(1)}, q.options().dtype(at::kFloat));
  fmha_fwd_params p = {};
  fill_common(p, q, k, v, o, scale > 0 ? scale : default_scale(q));
  p.lse = lse.data_ptr<float>();
  p.causal = is_causal ? 1 : 0;
  MaskLayout m;
  if (mask.has_value() && mask->defined()) {
    m = mask_layout(*mask, q, k.size(1), "mask");
    p.mask = m.t.data_ptr();
    p.mask_kind = FMHA_MASK_ADDITIVE;
    p.mask_bh_div = m.bh_div;
    p.mask_stride_b = m.stride_b;
    p.mask_stride_q = m.stride_q;
  }
  TORCH_CHECK(p_drop >= 0.0 && p_drop < 1.0, "mha_manual: p_drop must be in [0,1)");
  if (p_drop > 0.0) {
    p.drop_kind = FMHA_DROP_PHILOX;
    p.p_drop = static_cast<float>(p_drop);
    p.drop_scale = static_cast<float>(1.0 / (1.0 - p_drop));
    p.seed = static_cast<uint64_t>(seed);
    p.offset = static_cast<uint64_t>(offset);
  }
  at::Tensor kv_keep;
  set_kv_len(p, kv_len, q, kv_keep);
  launch_fwd(p, q);
  return std::make_tuple(o, lse);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor>
fmha_bwd(const at::Tensor &dout, const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
         const at::Tensor &o, const at::Tensor &lse, const c10::optional<at::Tensor> &mask, double scale,
         bool is_causal, double p_drop, int64_t seed, int64_t offset, const c10::optional<at::Tensor> &kv_len) {
  check_qkv(q, k, v);
  at::DeviceGuard guard(q.device());
  TORCH_CHECK(dout.is_cuda() && o.is_cuda() && lse.is_cuda(), "mha_manual: dout/o/lse must live on the GPU");
  TORCH_CHECK(dout.sizes() == q.sizes() && o.sizes() == q.sizes() && dout.scalar_type() == q.scalar_type() &&
                  o.scalar_type() == q.scalar_type(),
              "mha_manual: dout and o must match q in shape and dtype");
  TORCH_CHECK(lse.scalar_type() == at::kFloat && lse.dim() == 2 && lse.size(0) == q.size(0) &&
                  lse.size(1) == q.size(1),
              "mha_manual: lse must be float32 [BH,Sq]");
  at::Tensor doutc = dout.contiguous(), oc = o.contiguous(), lsec = lse.contiguous();
  at::Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v);
  at::Tensor delta = at::empty_like(lsec);
  fmha_bwd_params p = {};
  p.q = q.data_ptr();
  p.k = k.data_ptr();
  p.v = v.data_ptr();
  p.o = oc.data_ptr();
  p.dout = doutc.data_ptr();
  p.lse = lsec.data_ptr<float>();
  p.delta = delta.data_ptr<float>();
  p.dq = dq.data_ptr();
  p.dk = dk.data_ptr();
  p.dv = dv.data_ptr();
  p.bh = static_cast<int32_t>(q.size(0));
  p.sq = static_cast<int32_t>(q.size(1));
  p.sk = static_cast<int32_t>(k.size(1));
  p.d = static_cast<int32_t>(q.size(2));
  p.dtype = dtype_code(q);
  p.scale = static_cast<float>(scale > 0 ? scale : default_scale(q));
  p.causal = is_causal ? 1 : 0;
  MaskLayout m;
  if (mask.has_value() && mask->defined()) {
    m = mask_layout(*mask, q, k.size(1), "mask");
    p.mask = m.t.data_ptr();
    p.mask_kind = FMHA_MASK_ADDITIVE;
    p.mask_bh_div = m.bh_div;
    p.mask_stride_b = m.stride_b;
    p.mask_stride_q = m.stride_q;
  }
  TORCH_CHECK(p_drop >= 0.0 && p_drop < 1.0, "mha_manual: p_drop must be in [0,1)");
  if (p_drop > 0.0) {
    p.drop_kind = FMHA_DROP_PHILOX;
    p.p_drop = static_cast<float>(p_drop);
    p.drop_scale = static_cast<float>(1.0 / (1.0 - p_drop));
    p.seed = static_cast<uint64_t>(seed);
    p.offset = static_cast<uint64_t>(offset);
  }
  at::Tensor kv_keep;
  set_kv_len(p, kv_len, q, kv_keep);
  const int rc = fmha_bwd_launch(&p, current_stream(q));
  TORCH_CHECK(rc == FMHA_OK, "mha_manual backward: ", fmha_strerror(rc));
  return std::make_tuple(dq, dk, dv);
}

// uint8 [bh,sq,sk] keep decisions (1 keep / 0 drop) for (seed, offset, p_drop) on `like`'s device.
at::Tensor philox_keep_mask_op(const at::Tensor &like, int64_t bh, int64_t sq, int64_t sk, double p_drop,
                                 int64_t seed, int64_t offset) {
  TORCH_CHECK(like.is_cuda(), "mha_manual: `like` must live on the GPU");
  at::DeviceGuard guard(like.device());
  at::Tensor out = at::empty({bh, sq, sk}, like.options().dtype(at::kByte));
  const int rc = fmha_philox_keep_mask(static_cast<uint64_t>(seed), static_cast<uint64_t>(offset),
                                       static_cast<float>(p_drop), static_cast<int32_t>(bh),
                                       static_cast<int32_t>(sq), static_cast<int32_t>(sk),
                                       out.data_ptr<uint8_t>(), current_stream(like));
  TORCH_CHECK(rc == FMHA_OK, "mha_manual keep mask: ", fmha_strerror(rc));
  return out;
}

TORCH_LIBRARY(mha_manual, m) {
  m.def("fmha_nvfuser(Tensor input, Tensor qk, Tensor v, Tensor amask) -> Tensor");
  m.def("fmha_train_nvfuser(Tensor input, Tensor qk, Tensor v, Tensor pad_mask, Tensor dropout_mask) -> Tensor");
  m.def("fmha_train_saveim_nvfuser(Tensor input, Tensor qk, Tensor v, Tensor pad_mask, Tensor dropout_mask) -> "
        "Tensor[]");
  m.def("fmha_fwd(Tensor q, Tensor k, Tensor v, Tensor? mask, float scale, bool is_causal, float p_drop, int seed, "
        "int offset, Tensor? kv_len=None) -> (Tensor, Tensor)");
  m.def("fmha_bwd(Tensor dout, Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, Tensor? mask, float scale, bool "
        "is_causal, float p_drop, int seed, int offset, Tensor? kv_len=None) -> (Tensor, Tensor, Tensor)");
  m.def("fmha_philox_keep_mask(Tensor like, int bh, int sq, int sk, float p_drop, int seed, int offset) -> Tensor");
}

// On ROCm builds of PyTorch the CUDA dispatch key is the HIP device's key.
TORCH_LIBRARY_IMPL(mha_manual, CUDA, m) {
  m.impl("fmha_nvfuser", fmha_nvfuser);
  m.impl("fmha_train_nvfuser", fmha_train_nvfuser);
  m.impl("fmha_train_saveim_nvfuser", fmha_train_saveim_nvfuser);
  m.impl("fmha_fwd", fmha_fwd);
  m.impl("fmha_bwd", fmha_bwd);
  m.impl("fmha_philox_keep_mask", philox_keep_mask_op);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) { m.doc() = "gfx950 fused multi-head attention (operators live in torch.ops.mha_manual)"; }
