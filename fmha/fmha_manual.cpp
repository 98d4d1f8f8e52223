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
#include <torch/csrc/autograd/custom_function.h>
#include <torch/extension.h>

#include <algorithm>
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
MaskLayout mask_layout(const at::Tensor &mask_in, const at::Tensor &q, int64_t bh, int64_t sq, int64_t sk,
                       const char *what) {
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
  MaskLayout m = mask_layout(amask, input, input.size(0), input.size(1), qk.size(1), "amask");
  at::Tensor o = at::empty_like(input);
  fmha_fwd_params p = {};
  p.struct_bytes = sizeof p;
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
  MaskLayout m = mask_layout(pad_mask, input, input.size(0), input.size(1), sk, "pad_mask");
  TORCH_CHECK(dropout_mask.is_cuda() && dropout_mask.device() == input.device() &&
                  dropout_mask.scalar_type() == input.scalar_type() && dropout_mask.dim() == 3 &&
                  dropout_mask.size(0) == bh && dropout_mask.size(1) == sq && dropout_mask.size(2) == sk,
              "mha_manual: dropout_mask must be a [BH,Sq,Sk] tensor of q's dtype on q's device");
  at::Tensor dm = dropout_mask.contiguous();
  at::Tensor o = at::empty_like(input);
  fmha_fwd_params p = {};
  p.struct_bytes = sizeof p;
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
  at::Tensor lse; // scratch: with it the library derives the saved outputs from one forward launch
  if (save) {
    lse = at::empty({bh, sq}, input.options().dtype(at::kFloat));
    p.lse = lse.data_ptr<float>();
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

// One of q, k, v, o, dout as the C ABI sees it: folded contiguous [BH,S,D] (heads = 0), or a 4-d
// [B,H,S,D] tensor of any batch / head / row strides whose rows are contiguous (heads = H).
struct RowsOf {
  at::Tensor t; // the tensor itself, or a dense copy where its strides cannot be passed on
  int64_t bh = 0, s = 0, d = 0;
  int32_t heads = 0;
  int64_t st[3] = {0, 0, 0};
};

RowsOf rows_of(const at::Tensor &x, const char *what) {
  TORCH_CHECK(x.is_cuda(), "mha_manual: ", what, " must live on the GPU");
  TORCH_CHECK(x.dim() == 3 || x.dim() == 4, "mha_manual: ", what, " must be [B*H,S,D] or [B,H,S,D]");
  RowsOf r;
  if (x.dim() == 3) {
    r.t = x.contiguous();
    r.bh = x.size(0);
    r.s = x.size(1);
    r.d = x.size(2);
    return r;
  }
  bool ok = x.stride(3) == 1 && (reinterpret_cast<uintptr_t>(x.data_ptr()) & 15u) == 0;
  for (int i = 0; i < 3; ++i) ok = ok && x.stride(i) >= 0 && x.stride(i) % 8 == 0;
  ok = ok && x.stride(2) >= x.size(3) && x.stride(2) < (int64_t(1) << 24);
  r.t = ok ? x : x.contiguous();
  r.bh = x.size(0) * x.size(1);
  r.s = x.size(2);
  r.d = x.size(3);
  r.heads = static_cast<int32_t>(x.size(1));
  for (int i = 0; i < 3; ++i) r.st[i] = r.t.stride(i);
  return r;
}

// A new tensor of x's shape with x's order of dimensions in memory, but dense: a [B,H,S,D] view of
// [B,S,H,D] memory (or of a slice of a packed projection) gets fresh [B,S,H,D] memory.
at::Tensor empty_like_rows(const at::Tensor &x) {
  if (x.dim() != 4) return at::empty(x.sizes(), x.options());
  std::vector<int64_t> order{0, 1, 2, 3};
  std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) { return x.stride(a) > x.stride(b); });
  std::vector<int64_t> sizes(4), inv(4);
  for (int i = 0; i < 4; ++i) {
    sizes[i] = x.size(order[i]);
    inv[order[i]] = i;
  }
  return at::empty(sizes, x.options()).permute(inv);
}

// The kernels copy K and V tiles with one set of offsets: where their rows are not equally far
// apart, both are replaced by dense copies.
void same_row_pitch(RowsOf &k, RowsOf &v) {
  if (k.heads == 0 || v.heads == 0 || k.st[2] == v.st[2]) return;
  k = rows_of(k.t.contiguous(), "k");
  v = rows_of(v.t.contiguous(), "v");
}

void set_stride(int64_t (&dst)[3], const RowsOf &r) {
  for (int i = 0; i < 3; ++i) dst[i] = r.st[i];
}

void check_rows(const RowsOf &q, const RowsOf &k, const RowsOf &v) {
  TORCH_CHECK(q.t.scalar_type() == k.t.scalar_type() && q.t.scalar_type() == v.t.scalar_type(),
              "mha_manual: q/k/v must share one dtype");
  TORCH_CHECK(q.heads == k.heads && q.heads == v.heads, "mha_manual: q/k/v must be all 3-d or all 4-d with one H");
  TORCH_CHECK(k.bh == q.bh && v.bh == q.bh && k.d == q.d && v.d == q.d && v.s == k.s,
              "mha_manual: shapes must be q [..,Sq,D], k [..,Sk,D], v [..,Sk,D] over the same heads");
  TORCH_CHECK(k.t.device() == q.t.device() && v.t.device() == q.t.device(), "mha_manual: q/k/v on different devices");
}

// Optional valid key counts: an int32 vector of B entries on q's device, B dividing BH.
template <typename P> void set_kv_len(P &p, const c10::optional<at::Tensor> &kv_len, int64_t bh, at::Tensor &keep) {
  if (!kv_len.has_value() || !kv_len->defined()) return;
  TORCH_CHECK(kv_len->is_cuda() && kv_len->scalar_type() == at::kInt && kv_len->dim() == 1 && kv_len->numel() > 0 &&
                  bh % kv_len->numel() == 0,
              "mha_manual: kv_len must be an int32 GPU vector whose length divides BH");
  keep = kv_len->contiguous();
  p.kv_len = keep.data_ptr<int32_t>();
  p.kv_len_bh_div = static_cast<int32_t>(bh / keep.numel());
}

template <typename P>
void set_mask_and_dropout(P &p, MaskLayout &m, const c10::optional<at::Tensor> &mask, const RowsOf &q, int64_t sk,
                          double p_drop, int64_t seed, int64_t offset) {
  if (mask.has_value() && mask->defined()) {
    m = mask_layout(*mask, q.t, q.bh, q.s, sk, "mask");
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
    p.drop_scale = fmha_drop_scale(static_cast<float>(p_drop)); // keeps the mean at the realised keep probability
    p.seed = static_cast<uint64_t>(seed);
    p.offset = static_cast<uint64_t>(offset);
  }
}


// The C ABI takes any head dim that is a multiple of 8 up to 256 as it is (rows of whole 16-byte pieces:
// the kernels run at the next built size, 64 / 128 / 256, and neither read nor write the missing columns).
// Only head dims that are not multiples of 8 are zero-padded here, to the next multiple: zero columns add
// nothing to Q.K^T, the padded columns of V give zero columns of O (and zero columns of dO leave the other
// gradients untouched), so results are those of the original head dim, at the cost of a copy of every operand.
int64_t padded_head_dim(int64_t d) {
  TORCH_CHECK(d >= 1 && d <= 256, "mha_manual: head dim must be in [1, 256], got ", d);
  return (d + 7) / 8 * 8;
}
at::Tensor pad_head_dim(const at::Tensor &x, int64_t to) {
  return at::constant_pad_nd(x, {0, to - x.size(-1)}, 0);
}

// q, k, v: [B*H,S,D] contiguous (the reference's layout) or [B,H,S,D] views of any batch / head /
// row strides (e.g. x.view(B,S,H,D).transpose(1,2), or a slice of a packed QKV projection), read
// in place (any D up to 256; see above).  scale <= 0 selects 1/sqrt(D).  Dropout decisions come from Philox4x32-10 keyed by
// (seed, offset); p_drop == 0 disables dropout.  Returns (O, LSE fp32): O in q's shape and
// dimension order, LSE [B*H,Sq] or [B,H,Sq].
std::tuple<at::Tensor, at::Tensor> fmha_fwd(const at::Tensor &q_, const at::Tensor &k_, const at::Tensor &v_,
                                            const c10::optional<at::Tensor> &mask, double scale, bool is_causal,
                                            double p_drop, int64_t seed, int64_t offset,
                                            const c10::optional<at::Tensor> &kv_len) {
  TORCH_CHECK(q_.dim() >= 3 && k_.dim() == q_.dim() && v_.dim() == q_.dim() && k_.size(-1) == q_.size(-1) &&
                  v_.size(-1) == q_.size(-1),
              "mha_manual: q, k, v must be [B*H,S,D] or [B,H,S,D] with one head dim");
  if (const int64_t d = q_.size(-1), dp = padded_head_dim(d); dp != d) {
    auto [o, lse] = fmha_fwd(pad_head_dim(q_, dp), pad_head_dim(k_, dp), pad_head_dim(v_, dp), mask,
                             scale > 0 ? scale : 1.0 / std::sqrt(static_cast<double>(d)), is_causal, p_drop, seed,
                             offset, kv_len);
    return std::make_tuple(o.narrow(-1, 0, d).contiguous(), lse);
  }
  const RowsOf q = rows_of(q_, "q");
  RowsOf k = rows_of(k_, "k"), v = rows_of(v_, "v");
  same_row_pitch(k, v);
  check_rows(q, k, v);
  at::DeviceGuard guard(q.t.device());
  at::Tensor o = empty_like_rows(q.t);
  const RowsOf orow = rows_of(o, "o");
  at::Tensor lse = q.heads ? at::empty({q_.size(0), q_.size(1), q.s}, q.t.options().dtype(at::kFloat))
                           : at::empty({q.bh, q.s}, q.t.options().dtype(at::kFloat));
  fmha_fwd_params p = {};
  p.struct_bytes = sizeof p;
  p.q = q.t.data_ptr();
  p.k = k.t.data_ptr();
  p.v = v.t.data_ptr();
  p.o = o.data_ptr();
  p.bh = static_cast<int32_t>(q.bh);
  p.sq = static_cast<int32_t>(q.s);
  p.sk = static_cast<int32_t>(k.s);
  p.d = static_cast<int32_t>(q.d);
  p.dtype = dtype_code(q.t);
  p.scale = static_cast<float>(scale > 0 ? scale : 1.0 / std::sqrt(static_cast<double>(q.d)));
  p.heads = q.heads;
  set_stride(p.q_stride, q);
  set_stride(p.k_stride, k);
  set_stride(p.v_stride, v);
  set_stride(p.o_stride, orow);
  p.lse = lse.data_ptr<float>();
  p.causal = is_causal ? 1 : 0;
  MaskLayout m;
  set_mask_and_dropout(p, m, mask, q, k.s, p_drop, seed, offset);
  at::Tensor kv_keep;
  set_kv_len(p, kv_len, q.bh, kv_keep);
  // Few heads, few query rows and a long key range (decode steps): given room for the pieces' partial
  // results the library cuts the key range into pieces and fills the whole chip.
  at::Tensor workspace;
  if (const uint64_t need = fmha_fwd_workspace_bytes(&p); need > 0) {
    workspace = at::empty({static_cast<int64_t>(need)}, q.t.options().dtype(at::kByte));
    p.workspace = workspace.data_ptr();
    p.workspace_bytes = need;
  }
  launch_fwd(p, q.t);
  return std::make_tuple(o, lse);
}

// Gradients of fmha_fwd's inputs; tensors as there (dout and o in q's shape, any strides), lse as
// fmha_fwd returned it.  dq, dk, dv come back in the dimension order of q, k, v.
std::tuple<at::Tensor, at::Tensor, at::Tensor>
fmha_bwd(const at::Tensor &dout_, const at::Tensor &q_, const at::Tensor &k_, const at::Tensor &v_,
         const at::Tensor &o_, const at::Tensor &lse, const c10::optional<at::Tensor> &mask, double scale,
         bool is_causal, double p_drop, int64_t seed, int64_t offset, const c10::optional<at::Tensor> &kv_len) {
  TORCH_CHECK(q_.dim() >= 3 && k_.dim() == q_.dim() && v_.dim() == q_.dim() && k_.size(-1) == q_.size(-1) &&
                  v_.size(-1) == q_.size(-1) && dout_.sizes() == q_.sizes() && o_.sizes() == q_.sizes(),
              "mha_manual: q, k, v must be [B*H,S,D] or [B,H,S,D] with one head dim, dout and o shaped like q");
  if (const int64_t d = q_.size(-1), dp = padded_head_dim(d); dp != d) {
    auto [dq, dk, dv] = fmha_bwd(pad_head_dim(dout_, dp), pad_head_dim(q_, dp), pad_head_dim(k_, dp),
                                 pad_head_dim(v_, dp), pad_head_dim(o_, dp), lse, mask,
                                 scale > 0 ? scale : 1.0 / std::sqrt(static_cast<double>(d)), is_causal, p_drop, seed,
                                 offset, kv_len);
    return std::make_tuple(dq.narrow(-1, 0, d).contiguous(), dk.narrow(-1, 0, d).contiguous(),
                           dv.narrow(-1, 0, d).contiguous());
  }
  const RowsOf q = rows_of(q_, "q");
  RowsOf k = rows_of(k_, "k"), v = rows_of(v_, "v");
  same_row_pitch(k, v);
  check_rows(q, k, v);
  at::DeviceGuard guard(q.t.device());
  TORCH_CHECK(dout_.sizes() == q_.sizes() && o_.sizes() == q_.sizes() && dout_.scalar_type() == q.t.scalar_type() &&
                  o_.scalar_type() == q.t.scalar_type(),
              "mha_manual: dout and o must match q in shape and dtype");
  const RowsOf dout = rows_of(dout_, "dout"), o = rows_of(o_, "o");
  TORCH_CHECK(lse.is_cuda() && lse.scalar_type() == at::kFloat && lse.numel() == q.bh * q.s &&
                  lse.size(-1) == q.s,
              "mha_manual: lse must be float32 [BH,Sq] or [B,H,Sq]");
  at::Tensor lsec = lse.contiguous();
  at::Tensor dq = empty_like_rows(q.t), dk = empty_like_rows(k.t), dv = empty_like_rows(v.t);
  const RowsOf dqr = rows_of(dq, "dq"), dkr = rows_of(dk, "dk"), dvr = rows_of(dv, "dv");
  at::Tensor delta = at::empty_like(lsec);
  fmha_bwd_params p = {};
  p.struct_bytes = sizeof p;
  p.q = q.t.data_ptr();
  p.k = k.t.data_ptr();
  p.v = v.t.data_ptr();
  p.o = o.t.data_ptr();
  p.dout = dout.t.data_ptr();
  p.lse = lsec.data_ptr<float>();
  p.delta = delta.data_ptr<float>();
  p.dq = dq.data_ptr();
  p.dk = dk.data_ptr();
  p.dv = dv.data_ptr();
  p.bh = static_cast<int32_t>(q.bh);
  p.sq = static_cast<int32_t>(q.s);
  p.sk = static_cast<int32_t>(k.s);
  p.d = static_cast<int32_t>(q.d);
  p.dtype = dtype_code(q.t);
  p.scale = static_cast<float>(scale > 0 ? scale : 1.0 / std::sqrt(static_cast<double>(q.d)));
  p.causal = is_causal ? 1 : 0;
  p.heads = q.heads;
  set_stride(p.q_stride, q);
  set_stride(p.k_stride, k);
  set_stride(p.v_stride, v);
  set_stride(p.o_stride, o);
  set_stride(p.do_stride, dout);
  set_stride(p.dq_stride, dqr);
  set_stride(p.dk_stride, dkr);
  set_stride(p.dv_stride, dvr);
  MaskLayout m;
  set_mask_and_dropout(p, m, mask, q, k.s, p_drop, seed, offset);
  at::Tensor kv_keep;
  set_kv_len(p, kv_len, q.bh, kv_keep);
  const int rc = fmha_bwd_launch(&p, current_stream(q.t));
  TORCH_CHECK(rc == FMHA_OK, "mha_manual backward: ", fmha_strerror(rc));
  return std::make_tuple(dq, dk, dv);
}

// Forward on e4m3 inputs (torch.float8_e4m3fn, [B*H,S,D] contiguous, D = 64 or 128) with one dequantisation
// factor per tensor; O comes back as float16, or bfloat16 when out_bf16 (the dtype an optional per-key additive
// mask [B*H|B,1,Sk] / [B,1,1,Sk] must have).  Returns (O, LSE fp32).  Not in the reference (fp16 only).
std::tuple<at::Tensor, at::Tensor> fmha_fwd_fp8(const at::Tensor &q8, const at::Tensor &k8, const at::Tensor &v8,
                                                double descale_q, double descale_k, double descale_v,
                                                const c10::optional<at::Tensor> &mask, double scale, bool is_causal,
                                                bool out_bf16, const c10::optional<at::Tensor> &kv_len) {
  for (const at::Tensor *t : {&q8, &k8, &v8})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat8_e4m3fn && t->dim() == 3 && t->is_contiguous(),
                "mha_manual: q, k, v must be contiguous [B*H,S,D] float8_e4m3fn GPU tensors");
  TORCH_CHECK(k8.size(0) == q8.size(0) && v8.sizes() == k8.sizes() && k8.size(2) == q8.size(2),
              "mha_manual: shapes must be q [BH,Sq,D], k [BH,Sk,D], v [BH,Sk,D]");
  at::DeviceGuard guard(q8.device());
  const auto odt = out_bf16 ? at::kBFloat16 : at::kHalf;
  at::Tensor o = at::empty(q8.sizes(), q8.options().dtype(odt));
  at::Tensor lse = at::empty({q8.size(0), q8.size(1)}, q8.options().dtype(at::kFloat));
  fmha_fwd_fp8_params p = {};
  p.struct_bytes = sizeof p;
  p.q = q8.data_ptr();
  p.k = k8.data_ptr();
  p.v = v8.data_ptr();
  p.o = o.data_ptr();
  p.lse = lse.data_ptr<float>();
  p.bh = static_cast<int32_t>(q8.size(0));
  p.sq = static_cast<int32_t>(q8.size(1));
  p.sk = static_cast<int32_t>(k8.size(1));
  p.d = static_cast<int32_t>(q8.size(2));
  p.out_dtype = out_bf16 ? FMHA_DTYPE_BF16 : FMHA_DTYPE_F16;
  p.scale = static_cast<float>(scale > 0 ? scale : 1.0 / std::sqrt(static_cast<double>(q8.size(2))));
  p.descale_q = static_cast<float>(descale_q);
  p.descale_k = static_cast<float>(descale_k);
  p.descale_v = static_cast<float>(descale_v);
  p.causal = is_causal ? 1 : 0;
  MaskLayout m;
  if (mask.has_value() && mask->defined()) {
    m = mask_layout(*mask, o, q8.size(0), q8.size(1), k8.size(1), "mask");
    TORCH_CHECK(m.stride_q == 0, "mha_manual: the e4m3 forward takes per-key masks ([..,1,Sk]) only");
    p.mask = m.t.data_ptr();
    p.mask_bh_div = m.bh_div;
    p.mask_stride_b = m.stride_b;
  }
  // valid key counts and the key range in pieces: launches of one to four query rows (the decode kernel) only
  at::Tensor kv_keep, workspace;
  set_kv_len(p, kv_len, q8.size(0), kv_keep);
  if (const uint64_t need = fmha_fwd_fp8_workspace_bytes(&p); need > 0) {
    workspace = at::empty({static_cast<int64_t>(need)}, q8.options().dtype(at::kByte));
    p.workspace = workspace.data_ptr();
    p.workspace_bytes = need;
  }
  const int rc = fmha_fwd_fp8_launch(&p, current_stream(q8));
  TORCH_CHECK(rc == FMHA_OK, "mha_manual e4m3 forward: ", fmha_strerror(rc));
  return std::make_tuple(o, lse);
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

// Autograd formula of fmha_fwd (the reference registers none: fmha/fmha_manual.cpp:1240-1250, its perf runs
// are under no_grad): O is differentiable in q, k and v; the row log-sum-exp, the mask and the key counts
// are not.  Nothing of size S x S is kept for the backward: it recomputes P from the saved LSE and
// regenerates the dropout decisions from the same (seed, offset).
class FmhaFunction : public torch::autograd::Function<FmhaFunction> {
 public:
  static torch::autograd::variable_list forward(torch::autograd::AutogradContext *ctx, const at::Tensor &q,
                                                const at::Tensor &k, const at::Tensor &v,
                                                const c10::optional<at::Tensor> &mask, double scale, bool is_causal,
                                                double p_drop, int64_t seed, int64_t offset,
                                                const c10::optional<at::Tensor> &kv_len) {
    at::AutoDispatchBelowADInplaceOrView below;
    auto [o, lse] = fmha_fwd(q, k, v, mask, scale, is_causal, p_drop, seed, offset, kv_len);
    const bool has_mask = mask.has_value() && mask->defined(), has_len = kv_len.has_value() && kv_len->defined();
    ctx->save_for_backward({q, k, v, o, lse, has_mask ? *mask : at::empty({0}, q.options()),
                            has_len ? *kv_len : at::empty({0}, q.options().dtype(at::kInt))});
    ctx->saved_data["has_mask"] = has_mask;
    ctx->saved_data["has_len"] = has_len;
    ctx->saved_data["scale"] = scale;
    ctx->saved_data["is_causal"] = is_causal;
    ctx->saved_data["p_drop"] = p_drop;
    ctx->saved_data["seed"] = seed;
    ctx->saved_data["offset"] = offset;
    ctx->mark_non_differentiable({lse});
    return {o, lse};
  }
  static torch::autograd::variable_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    const at::Tensor &q = saved[0], &k = saved[1], &v = saved[2], &o = saved[3], &lse = saved[4];
    const at::Tensor dout = grads[0].defined() ? grads[0] : at::zeros_like(o);
    c10::optional<at::Tensor> mask, kv_len;
    if (ctx->saved_data["has_mask"].toBool()) mask = saved[5];
    if (ctx->saved_data["has_len"].toBool()) kv_len = saved[6];
    auto [dq, dk, dv] = fmha_bwd(dout, q, k, v, o, lse, mask, ctx->saved_data["scale"].toDouble(),
                                 ctx->saved_data["is_causal"].toBool(), ctx->saved_data["p_drop"].toDouble(),
                                 ctx->saved_data["seed"].toInt(), ctx->saved_data["offset"].toInt(), kv_len);
    at::Tensor none;
    return {dq, dk, dv, none, none, none, none, none, none, none};
  }
};

std::tuple<at::Tensor, at::Tensor> fmha_fwd_autograd(const at::Tensor &q, const at::Tensor &k, const at::Tensor &v,
                                                     const c10::optional<at::Tensor> &mask, double scale,
                                                     bool is_causal, double p_drop, int64_t seed, int64_t offset,
                                                     const c10::optional<at::Tensor> &kv_len) {
  auto r = FmhaFunction::apply(q, k, v, mask, scale, is_causal, p_drop, seed, offset, kv_len);
  return std::make_tuple(r[0], r[1]);
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
  m.def("fmha_fwd_fp8(Tensor q8, Tensor k8, Tensor v8, float descale_q, float descale_k, float descale_v, Tensor? mask, "
        "float scale, bool is_causal, bool out_bf16=False, Tensor? kv_len=None) -> (Tensor, Tensor)");
}

// On ROCm builds of PyTorch the CUDA dispatch key is the HIP device's key.
TORCH_LIBRARY_IMPL(mha_manual, CUDA, m) {
  m.impl("fmha_nvfuser", fmha_nvfuser);
  m.impl("fmha_train_nvfuser", fmha_train_nvfuser);
  m.impl("fmha_train_saveim_nvfuser", fmha_train_saveim_nvfuser);
  m.impl("fmha_fwd", fmha_fwd);
  m.impl("fmha_bwd", fmha_bwd);
  m.impl("fmha_philox_keep_mask", philox_keep_mask_op);
  m.impl("fmha_fwd_fp8", fmha_fwd_fp8);
}

// fmha_fwd is differentiable by itself; the other operators stay without a formula, like the reference's.
TORCH_LIBRARY_IMPL(mha_manual, Autograd, m) { m.impl("fmha_fwd", fmha_fwd_autograd); }

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) { m.doc() = "gfx950 fused multi-head attention (operators live in torch.ops.mha_manual)"; }
