// XLA typed-FFI handlers over the plain C ABI (include/mi355_w8a8.h).
//
// Built only where jaxlib's headers exist (xla/ffi/api/ffi.h ships inside jaxlib/include);
// the build script skips this file otherwise.  Handler shape follows the reference's
// skyrl/tx/kernels/rocm/ffi/gdn_ffi_smoke.hip:43-82 and its W8A8 design note
// rocm/QUANTIZED_FFI.md:589-614: typed buffers in, result buffers out (the workspace is an
// explicit result so XLA owns its stream-ordered lifetime), the platform stream from the call
// context, validation -> InvalidArgument, launch failure -> Internal, no synchronisation.
#if __has_include("xla/ffi/api/ffi.h")
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/mi355_w8a8.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error ToError(int status, const char* what) {
  if (status == MI355_W8A8_OK) return ffi::Error::Success();
  if (status == MI355_W8A8_ERR_LAUNCH) return ffi::Error::Internal(what);
  return ffi::Error::InvalidArgument(mi355_w8a8_status_string(status));
}

bool RowsAndK(ffi::Span<const int64_t> dims, uint32_t* m, uint32_t* k) {
  if (dims.size() < 2) return false;
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < dims.size(); ++i) rows *= dims[i];
  if (rows <= 0 || rows > (1 << 20) || dims.back() <= 0 || dims.back() > 16384) return false;
  *m = static_cast<uint32_t>(rows);
  *k = static_cast<uint32_t>(dims.back());
  return true;
}

// x [.., K] bf16, packed weight u8 [bytes], scales f32 [N], A bf16 [n, K, r], B bf16 [n, r, N],
// scaling f32 [n], adapter index s32 [M]; optional stage inputs are passed as size-0 buffers
// when unused.  Results: y bf16 [.., n_out], workspace u8 [mi355_w8a8_workspace_bytes].
ffi::Error Forward(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::U8> w_packed,
                   ffi::Buffer<ffi::F32> w_scales, ffi::Buffer<ffi::BF16> lora_a,
                   ffi::Buffer<ffi::BF16> lora_b, ffi::Buffer<ffi::F32> lora_scaling,
                   ffi::Buffer<ffi::S32> adapter_indices, ffi::Buffer<ffi::F32> rms_gamma,
                   ffi::Buffer<ffi::BF16> residual, ffi::ResultBuffer<ffi::BF16> y,
                   ffi::ResultBuffer<ffi::U8> workspace, int32_t swiglu, float rms_eps, int32_t entry) {
  mi355_w8a8_problem p{};
  p.struct_size = sizeof(p);
  if (!RowsAndK(x.dimensions(), &p.m, &p.k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  if (w_scales.dimensions().size() != 1) return ffi::Error::InvalidArgument("w_scales must be f32 [N]");
  p.n = static_cast<uint32_t>(w_scales.dimensions()[0]);
  if (w_packed.size_bytes() != mi355_w8a8_packed_weight_bytes(p.k, p.n))
    return ffi::Error::InvalidArgument("packed weight size does not match (K, N)");
  const bool lora = lora_a.element_count() > 0;
  if (lora) {
    auto da = lora_a.dimensions();
    auto db = lora_b.dimensions();
    if (da.size() != 3 || db.size() != 3 || da[1] != p.k || db[0] != da[0] || db[1] != da[2] ||
        db[2] != p.n || lora_scaling.element_count() != static_cast<size_t>(da[0]))
      return ffi::Error::InvalidArgument("LoRA A/B/scaling must be [n,K,r], [n,r,N], [n]");
    p.n_adapters = static_cast<uint32_t>(da[0]);
    p.rank = static_cast<uint32_t>(da[2]);
    p.lora_a = lora_a.untyped_data();
    p.lora_b = lora_b.untyped_data();
    p.lora_scaling = lora_scaling.typed_data();
    if (adapter_indices.element_count() > 0) {
      if (adapter_indices.element_count() != p.m)
        return ffi::Error::InvalidArgument("adapter_indices must hold one entry per row");
      p.adapter_indices = adapter_indices.typed_data();
    }
  }
  if (rms_gamma.element_count() > 0) {
    if (rms_gamma.element_count() != p.k) return ffi::Error::InvalidArgument("rms_gamma must be f32 [K]");
    p.rms_gamma = rms_gamma.typed_data();
    p.rms_eps = rms_eps;
  }
  const uint32_t n_out = swiglu ? p.n / 2 : p.n;
  if (y->element_count() != static_cast<size_t>(p.m) * n_out)
    return ffi::Error::InvalidArgument("result must be bf16 [..., n_out]");
  if (residual.element_count() > 0) {
    if (residual.element_count() != y->element_count())
      return ffi::Error::InvalidArgument("residual must match the result shape");
    p.residual = residual.untyped_data();
  }
  p.flags = swiglu ? MI355_W8A8_FLAG_SWIGLU : 0u;
  p.x = x.untyped_data();
  p.w_packed = w_packed.untyped_data();
  p.w_scales = w_scales.typed_data();
  p.out = y->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  int status;
  switch (entry) {
    case 1: status = mi355_w8a8_lora_linear_v1(&p, stream); break;
    case 2: status = mi355_w8a8_rms_gateup_swiglu_v1(&p, stream); break;
    case 3: status = mi355_w8a8_lora_residual_v1(&p, stream); break;
    default: status = mi355_w8a8_forward_v1(&p, stream); break;
  }
  return ToError(status, "mi355_w8a8 forward launch submission failed");
}

// Backward of the plain linear.  x [.., K] bf16, dy [.., N] bf16, packed weight, scales, A, B,
// scaling and adapter index as in Forward (size-0 buffers when there is no LoRA).  Results:
// dx bf16 [.., K], dA bf16 [n, K, r], dB bf16 [n, r, N], dscaling f32 [n] (size-0 without LoRA),
// workspace u8 [mi355_w8a8_bwd_workspace_bytes].
ffi::Error Backward(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::BF16> dy,
                    ffi::Buffer<ffi::U8> w_packed, ffi::Buffer<ffi::F32> w_scales,
                    ffi::Buffer<ffi::BF16> lora_a, ffi::Buffer<ffi::BF16> lora_b,
                    ffi::Buffer<ffi::F32> lora_scaling, ffi::Buffer<ffi::S32> adapter_indices,
                    ffi::ResultBuffer<ffi::BF16> dx, ffi::ResultBuffer<ffi::BF16> d_lora_a,
                    ffi::ResultBuffer<ffi::BF16> d_lora_b, ffi::ResultBuffer<ffi::F32> d_lora_scaling,
                    ffi::ResultBuffer<ffi::U8> workspace) {
  mi355_w8a8_bwd_problem p{};
  p.struct_size = sizeof(p);
  if (!RowsAndK(x.dimensions(), &p.m, &p.k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  if (w_scales.dimensions().size() != 1) return ffi::Error::InvalidArgument("w_scales must be f32 [N]");
  p.n = static_cast<uint32_t>(w_scales.dimensions()[0]);
  auto ddy = dy.dimensions();
  if (ddy.size() < 2 || ddy.back() != p.n || dy.element_count() != static_cast<size_t>(p.m) * p.n)
    return ffi::Error::InvalidArgument("dy must be bf16 [..., N] over the rows of x");
  if (w_packed.size_bytes() != mi355_w8a8_packed_weight_bytes(p.k, p.n))
    return ffi::Error::InvalidArgument("packed weight size does not match (K, N)");
  if (dx->element_count() != x.element_count()) return ffi::Error::InvalidArgument("dx must match x");
  if (lora_a.element_count() > 0) {
    auto da = lora_a.dimensions();
    auto db = lora_b.dimensions();
    if (da.size() != 3 || db.size() != 3 || da[1] != p.k || db[0] != da[0] || db[1] != da[2] ||
        db[2] != p.n || lora_scaling.element_count() != static_cast<size_t>(da[0]))
      return ffi::Error::InvalidArgument("LoRA A/B/scaling must be [n,K,r], [n,r,N], [n]");
    if (d_lora_a->element_count() != lora_a.element_count() || d_lora_b->element_count() != lora_b.element_count() ||
        d_lora_scaling->element_count() != lora_scaling.element_count())
      return ffi::Error::InvalidArgument("the LoRA cotangents must match the LoRA parameters");
    p.n_adapters = static_cast<uint32_t>(da[0]);
    p.rank = static_cast<uint32_t>(da[2]);
    p.lora_a = lora_a.untyped_data();
    p.lora_b = lora_b.untyped_data();
    p.lora_scaling = lora_scaling.typed_data();
    p.d_lora_a = d_lora_a->untyped_data();
    p.d_lora_b = d_lora_b->untyped_data();
    p.d_lora_scaling = d_lora_scaling->typed_data();
    if (adapter_indices.element_count() > 0) {
      if (adapter_indices.element_count() != p.m)
        return ffi::Error::InvalidArgument("adapter_indices must hold one entry per row");
      p.adapter_indices = adapter_indices.typed_data();
    }
  }
  p.x = x.untyped_data();
  p.dy = dy.untyped_data();
  p.w_packed = w_packed.untyped_data();
  p.w_scales = w_scales.typed_data();
  p.dx = dx->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  return ToError(mi355_w8a8_lora_linear_bwd_v1(&p, stream), "mi355_w8a8 backward launch submission failed");
}

ffi::Error QuantizeRows(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::ResultBuffer<ffi::S8> codes,
                        ffi::ResultBuffer<ffi::F32> scales) {
  uint32_t m = 0, k = 0;
  if (!RowsAndK(x.dimensions(), &m, &k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  if (codes->element_count() != x.element_count() || scales->element_count() != m)
    return ffi::Error::InvalidArgument("codes must match x and scales must hold one value per row");
  return ToError(mi355_w8a8_quantize_rows_v1(x.untyped_data(), codes->typed_data(), scales->typed_data(), m, k,
                                             stream),
                 "mi355_w8a8 quantize launch submission failed");
}

ffi::Error PackWeight(hipStream_t stream, ffi::Buffer<ffi::S8> codes, ffi::ResultBuffer<ffi::U8> packed) {
  auto d = codes.dimensions();
  if (d.size() != 2 || d[0] <= 0 || d[1] <= 0) return ffi::Error::InvalidArgument("codes must be s8 [K, N]");
  const uint32_t k = static_cast<uint32_t>(d[0]), n = static_cast<uint32_t>(d[1]);
  if (packed->size_bytes() != mi355_w8a8_packed_weight_bytes(k, n))
    return ffi::Error::InvalidArgument("packed buffer size does not match (K, N)");
  return ToError(mi355_w8a8_pack_weight_v1(codes.typed_data(), packed->untyped_data(), k, n, stream),
                 "mi355_w8a8 pack launch submission failed");
}

// d_fused = swiglu pull-back(fused, d_product); fused bf16 [.., N], d_product bf16 [.., N / 2].
ffi::Error SwigluBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> fused, ffi::Buffer<ffi::BF16> d_product,
                     ffi::ResultBuffer<ffi::BF16> d_fused) {
  uint32_t m = 0, n = 0;
  if (!RowsAndK(fused.dimensions(), &m, &n))
    return ffi::Error::InvalidArgument("fused must be bf16 [..., N] with a non-empty row domain");
  if (d_product.element_count() * 2 != fused.element_count() || d_fused->element_count() != fused.element_count())
    return ffi::Error::InvalidArgument("d_product must be [..., N / 2] and d_fused must match fused");
  return ToError(mi355_w8a8_swiglu_bwd_v1(fused.untyped_data(), d_product.untyped_data(), d_fused->untyped_data(), m, n,
                                          stream),
                 "mi355_w8a8 swiglu pull-back launch submission failed");
}

// d_x = RMSNorm pull-back(x, gamma, d_normalized); x and d_normalized bf16 [.., K], gamma f32 [K].
ffi::Error RmsNormBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::F32> gamma,
                      ffi::Buffer<ffi::BF16> d_normalized, ffi::ResultBuffer<ffi::BF16> d_x, float eps) {
  uint32_t m = 0, k = 0;
  if (!RowsAndK(x.dimensions(), &m, &k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  if (gamma.element_count() != k || d_normalized.element_count() != x.element_count() ||
      d_x->element_count() != x.element_count())
    return ffi::Error::InvalidArgument("gamma must be f32 [K]; d_normalized and d_x must match x");
  return ToError(mi355_w8a8_rms_norm_bwd_v1(x.untyped_data(), gamma.typed_data(), d_normalized.untyped_data(),
                                            d_x->untyped_data(), m, k, eps, stream),
                 "mi355_w8a8 rms norm pull-back launch submission failed");
}

// router_logits f32 [T, E] -> weights f32 [T, top_k], selected s32 [T, top_k].
ffi::Error MoeRoute(hipStream_t stream, ffi::Buffer<ffi::F32> router_logits, ffi::ResultBuffer<ffi::F32> weights,
                    ffi::ResultBuffer<ffi::S32> selected, int32_t norm_topk_prob) {
  auto d = router_logits.dimensions();
  auto dw = weights->dimensions();
  if (d.size() != 2 || dw.size() != 2 || d[0] <= 0 || dw[0] != d[0] || dw[1] <= 0 ||
      selected->element_count() != weights->element_count())
    return ffi::Error::InvalidArgument("router_logits must be f32 [T, E]; weights and selected [T, top_k]");
  return ToError(mi355_w8a8_moe_route_v1(router_logits.typed_data(), static_cast<uint32_t>(d[0]),
                                         static_cast<uint32_t>(d[1]), static_cast<uint32_t>(dw[1]),
                                         norm_topk_prob ? 1u : 0u, weights->typed_data(), selected->typed_data(), stream),
                 "mi355_w8a8 moe route launch submission failed");
}

// Stable sort of the pairs by group.  tokens bf16 [P / repeat, H] (size 0: indices only), indices s32
// [P], adapter_indices s32 [P / repeat] (size 0: none).  Results: sorted_tokens bf16 [P, H] (size 0
// without tokens), group_sizes s32 [G], sort_indices and unsort_indices s32 [P], sorted_adapters s32
// [P] (size 0 without adapter indices), workspace u8 [mi355_w8a8_moe_dispatch_workspace_bytes].
ffi::Error MoeDispatch(hipStream_t stream, ffi::Buffer<ffi::BF16> tokens, ffi::Buffer<ffi::S32> indices,
                       ffi::Buffer<ffi::S32> adapter_indices, ffi::ResultBuffer<ffi::BF16> sorted_tokens,
                       ffi::ResultBuffer<ffi::S32> group_sizes, ffi::ResultBuffer<ffi::S32> sort_indices,
                       ffi::ResultBuffer<ffi::S32> unsort_indices, ffi::ResultBuffer<ffi::S32> sorted_adapters,
                       ffi::ResultBuffer<ffi::U8> workspace, int32_t repeat) {
  mi355_w8a8_moe_dispatch_problem p{};
  p.struct_size = sizeof(p);
  p.n_pairs = static_cast<uint32_t>(indices.element_count());
  p.n_groups = static_cast<uint32_t>(group_sizes->element_count());
  p.repeat = repeat > 0 ? static_cast<uint32_t>(repeat) : 0u;
  if (p.n_pairs == 0 || p.repeat == 0 || sort_indices->element_count() != p.n_pairs ||
      unsort_indices->element_count() != p.n_pairs)
    return ffi::Error::InvalidArgument("indices, sort_indices and unsort_indices must hold one entry per pair");
  if (tokens.element_count() > 0) {
    auto d = tokens.dimensions();
    if (d.size() != 2 || static_cast<uint64_t>(d[0]) * p.repeat != p.n_pairs ||
        sorted_tokens->element_count() != static_cast<size_t>(p.n_pairs) * d[1])
      return ffi::Error::InvalidArgument("tokens must be bf16 [P / repeat, H] and sorted_tokens [P, H]");
    p.width = static_cast<uint32_t>(d[1]);
    p.tokens = tokens.untyped_data();
    p.sorted_tokens = sorted_tokens->untyped_data();
  }
  if (adapter_indices.element_count() > 0) {
    if (adapter_indices.element_count() * p.repeat != p.n_pairs || sorted_adapters->element_count() != p.n_pairs)
      return ffi::Error::InvalidArgument("adapter_indices must be [P / repeat] and sorted_adapters [P]");
    p.adapter_indices = adapter_indices.typed_data();
    p.sorted_adapters = sorted_adapters->typed_data();
  }
  p.indices = indices.typed_data();
  p.group_sizes = group_sizes->typed_data();
  p.sort_indices = sort_indices->typed_data();
  p.unsort_indices = unsort_indices->typed_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  return ToError(mi355_w8a8_moe_dispatch_v1(&p, stream), "mi355_w8a8 moe dispatch launch submission failed");
}

// out[t] = sum_j expert_out[unsort[t k + j]] * weights[t, j]; expert_out bf16 [T k, H], out bf16 [T, H].
ffi::Error MoeCombine(hipStream_t stream, ffi::Buffer<ffi::BF16> expert_out, ffi::Buffer<ffi::S32> unsort_indices,
                      ffi::Buffer<ffi::F32> weights, ffi::ResultBuffer<ffi::BF16> out) {
  auto de = expert_out.dimensions();
  auto dw = weights.dimensions();
  if (de.size() != 2 || dw.size() != 2 || dw[0] <= 0 || dw[1] <= 0 || de[0] != dw[0] * dw[1] ||
      unsort_indices.element_count() != static_cast<size_t>(de[0]) ||
      out->element_count() != static_cast<size_t>(dw[0]) * de[1])
    return ffi::Error::InvalidArgument("expert_out must be [T * top_k, H], weights [T, top_k], out [T, H]");
  return ToError(mi355_w8a8_moe_combine_v1(expert_out.untyped_data(), unsort_indices.typed_data(), weights.typed_data(),
                                           out->untyped_data(), static_cast<uint32_t>(dw[0]),
                                           static_cast<uint32_t>(dw[1]), static_cast<uint32_t>(de[1]), stream),
                 "mi355_w8a8 moe combine launch submission failed");
}

// Grouped (ragged) call over rows already sorted by group: x bf16 [M or tokens, K], packed weights u8
// [n_weights * bytes], scales f32 [n_weights, N], A bf16 [G, K, r], B bf16 [G, r, N], scaling f32 [G]
// (size-0 buffers without LoRA), group_sizes s32 [G], x_row_map s32 [M] (size 0: row i of the call is
// row i of x).  Results: y bf16 [M, n_out], workspace u8 [mi355_w8a8_grouped_workspace_bytes].
ffi::Error Grouped(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::U8> w_packed,
                   ffi::Buffer<ffi::F32> w_scales, ffi::Buffer<ffi::BF16> lora_a, ffi::Buffer<ffi::BF16> lora_b,
                   ffi::Buffer<ffi::F32> lora_scaling, ffi::Buffer<ffi::S32> group_sizes,
                   ffi::Buffer<ffi::S32> x_row_map, ffi::ResultBuffer<ffi::BF16> y,
                   ffi::ResultBuffer<ffi::U8> workspace, int32_t swiglu, int32_t x_row_repeat) {
  mi355_w8a8_grouped_problem p{};
  p.struct_size = sizeof(p);
  uint32_t x_rows = 0;
  if (!RowsAndK(x.dimensions(), &x_rows, &p.k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  auto ds = w_scales.dimensions();
  if (ds.size() != 2 || ds[0] <= 0 || ds[1] <= 0) return ffi::Error::InvalidArgument("w_scales must be f32 [n_weights, N]");
  const uint32_t n_weights = static_cast<uint32_t>(ds[0]);
  p.n = static_cast<uint32_t>(ds[1]);
  p.n_groups = static_cast<uint32_t>(group_sizes.element_count());
  if (p.n_groups == 0 || p.n_groups % n_weights != 0)
    return ffi::Error::InvalidArgument("group_sizes must be s32 [G] with G a multiple of the number of weights");
  p.groups_per_weight = p.n_groups / n_weights;
  if (w_packed.size_bytes() != static_cast<size_t>(n_weights) * mi355_w8a8_packed_weight_bytes(p.k, p.n))
    return ffi::Error::InvalidArgument("packed weights do not match (n_weights, K, N)");
  if (x_row_map.element_count() > 0) {
    if (x_row_repeat < 1) return ffi::Error::InvalidArgument("x_row_repeat must be >= 1 with a row map");
    p.m = static_cast<uint32_t>(x_row_map.element_count());
    if (static_cast<uint64_t>(x_rows) * static_cast<uint32_t>(x_row_repeat) < p.m)
      return ffi::Error::InvalidArgument("x_row_map must not name more rows than x holds times x_row_repeat");
    p.x_row_map = x_row_map.typed_data();
    p.x_row_repeat = static_cast<uint32_t>(x_row_repeat);
    p.x_rows = x_rows;
  } else {
    p.m = x_rows;
  }
  if (lora_a.element_count() > 0) {
    auto da = lora_a.dimensions();
    auto db = lora_b.dimensions();
    if (da.size() != 3 || db.size() != 3 || da[0] != p.n_groups || da[1] != p.k || db[0] != da[0] ||
        db[1] != da[2] || db[2] != p.n || lora_scaling.element_count() != p.n_groups)
      return ffi::Error::InvalidArgument("LoRA A/B/scaling must be [G,K,r], [G,r,N], [G]");
    p.rank = static_cast<uint32_t>(da[2]);
    p.lora_a = lora_a.untyped_data();
    p.lora_b = lora_b.untyped_data();
    p.lora_scaling = lora_scaling.typed_data();
  }
  const uint32_t n_out = swiglu ? p.n / 2 : p.n;
  if (y->element_count() != static_cast<size_t>(p.m) * n_out)
    return ffi::Error::InvalidArgument("result must be bf16 [M, n_out]");
  p.flags = swiglu ? MI355_W8A8_FLAG_SWIGLU : 0u;
  p.x = x.untyped_data();
  p.w_packed = w_packed.untyped_data();
  p.w_scales = w_scales.typed_data();
  p.group_sizes = group_sizes.typed_data();
  p.out = y->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  return ToError(mi355_w8a8_grouped_v1(&p, stream), "mi355_w8a8 grouped launch submission failed");
}

// Attention input stage behind the fused QKV projection: fused bf16 [M, H 2 D + 2 Hkv D], the two
// head-norm weights f32 [D] (delta form), positions s32 [M].  Results: q bf16 [M, H, D], k and v bf16
// [M, Hkv, D], gate bf16 [M, H D].
ffi::Error QkvSplitNormRope(hipStream_t stream, ffi::Buffer<ffi::BF16> fused, ffi::Buffer<ffi::F32> q_norm_weight,
                            ffi::Buffer<ffi::F32> k_norm_weight, ffi::Buffer<ffi::S32> positions,
                            ffi::ResultBuffer<ffi::BF16> q, ffi::ResultBuffer<ffi::BF16> k,
                            ffi::ResultBuffer<ffi::BF16> v, ffi::ResultBuffer<ffi::BF16> gate, int32_t rotary_dim,
                            float rope_theta, float rms_eps) {
  mi355_w8a8_qkv_post_problem p{};
  p.struct_size = sizeof(p);
  auto dq = q->dimensions();
  auto dk = k->dimensions();
  if (dq.size() != 3 || dk.size() != 3 || dq[0] <= 0 || dk[0] != dq[0] || dk[2] != dq[2] || dq[1] <= 0 || dk[1] <= 0)
    return ffi::Error::InvalidArgument("q must be bf16 [M, H, D] and k bf16 [M, Hkv, D]");
  p.m = static_cast<uint32_t>(dq[0]);
  p.num_query_heads = static_cast<uint32_t>(dq[1]);
  p.num_kv_heads = static_cast<uint32_t>(dk[1]);
  p.head_dim = static_cast<uint32_t>(dq[2]);
  const size_t width = static_cast<size_t>(p.num_query_heads) * 2 * p.head_dim + 2 * static_cast<size_t>(p.num_kv_heads) * p.head_dim;
  if (fused.element_count() != static_cast<size_t>(p.m) * width || v->element_count() != k->element_count() ||
      gate->element_count() != q->element_count() || positions.element_count() != p.m ||
      q_norm_weight.element_count() != p.head_dim || k_norm_weight.element_count() != p.head_dim)
    return ffi::Error::InvalidArgument("fused, v, gate, positions or the norm weights do not match (M, H, Hkv, D)");
  if (rotary_dim < 0) return ffi::Error::InvalidArgument("rotary_dim must be >= 0");
  p.rotary_dim = static_cast<uint32_t>(rotary_dim);
  p.rope_theta = rope_theta;
  p.rms_eps = rms_eps;
  p.fused = fused.untyped_data();
  p.q_norm_weight = q_norm_weight.typed_data();
  p.k_norm_weight = k_norm_weight.typed_data();
  p.positions = positions.typed_data();
  p.q = q->untyped_data();
  p.k = k->untyped_data();
  p.v = v->untyped_data();
  p.gate = gate->untyped_data();
  return ToError(mi355_w8a8_qkv_split_norm_rope_v1(&p, stream), "mi355_w8a8 qkv stage launch submission failed");
}

// Group-scaled weight codes into the kernel's operand order: codes s8 [K_pad, N] (4-bit codes one per
// byte) -> packed u8 [mi355_w8a8_gq_packed_weight_bytes].
ffi::Error GqPackWeight(hipStream_t stream, ffi::Buffer<ffi::S8> codes, ffi::ResultBuffer<ffi::U8> packed,
                        int32_t weight_bits) {
  auto d = codes.dimensions();
  if (d.size() != 2 || d[0] <= 0 || d[1] <= 0) return ffi::Error::InvalidArgument("codes must be s8 [K_pad, N]");
  const uint32_t k_pad = static_cast<uint32_t>(d[0]), n = static_cast<uint32_t>(d[1]);
  const uint64_t need = mi355_w8a8_gq_packed_weight_bytes(k_pad, n, static_cast<uint32_t>(weight_bits));
  if (need == 0 || packed->size_bytes() != need)
    return ffi::Error::InvalidArgument("packed buffer size does not match (K_pad, N, weight_bits)");
  return ToError(mi355_w8a8_gq_pack_weight_v1(codes.typed_data(), packed->untyped_data(), k_pad, n,
                                              static_cast<uint32_t>(weight_bits), stream),
                 "mi355_w8a8 gq pack launch submission failed");
}

// Group-scaled linear (W4 / W8 codes, A4 / A8 activations, one scale per K group): x bf16 [.., K], packed
// weight, scales f32 [K_pad / group_size, N], LoRA as in Forward.  Results: y bf16 [.., N], workspace u8
// [mi355_w8a8_gq_workspace_bytes].
ffi::Error GqLinear(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::U8> w_packed,
                    ffi::Buffer<ffi::F32> w_scales, ffi::Buffer<ffi::BF16> lora_a, ffi::Buffer<ffi::BF16> lora_b,
                    ffi::Buffer<ffi::F32> lora_scaling, ffi::Buffer<ffi::S32> adapter_indices,
                    ffi::ResultBuffer<ffi::BF16> y, ffi::ResultBuffer<ffi::U8> workspace, int32_t group_size,
                    int32_t weight_bits, int32_t activation_bits) {
  mi355_w8a8_gq_problem p{};
  p.struct_size = sizeof(p);
  if (!RowsAndK(x.dimensions(), &p.m, &p.k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  auto ds = w_scales.dimensions();
  if (ds.size() != 2 || ds[0] <= 0 || ds[1] <= 0 || group_size <= 0)
    return ffi::Error::InvalidArgument("w_scales must be f32 [K_pad / group_size, N] and group_size positive");
  p.group_size = static_cast<uint32_t>(group_size);
  p.k_pad = static_cast<uint32_t>(ds[0]) * p.group_size;
  p.n = static_cast<uint32_t>(ds[1]);
  p.weight_bits = static_cast<uint32_t>(weight_bits);
  p.activation_bits = static_cast<uint32_t>(activation_bits);
  if (p.k_pad < p.k) return ffi::Error::InvalidArgument("the scale groups must cover K");
  const uint64_t need = mi355_w8a8_gq_packed_weight_bytes(p.k_pad, p.n, p.weight_bits);
  if (need == 0 || w_packed.size_bytes() != need)
    return ffi::Error::InvalidArgument("packed weight size does not match (K_pad, N, weight_bits)");
  if (lora_a.element_count() > 0) {
    auto da = lora_a.dimensions();
    auto db = lora_b.dimensions();
    if (da.size() != 3 || db.size() != 3 || da[1] != p.k || db[0] != da[0] || db[1] != da[2] || db[2] != p.n ||
        lora_scaling.element_count() != static_cast<size_t>(da[0]))
      return ffi::Error::InvalidArgument("LoRA A/B/scaling must be [n,K,r], [n,r,N], [n]");
    p.n_adapters = static_cast<uint32_t>(da[0]);
    p.rank = static_cast<uint32_t>(da[2]);
    p.lora_a = lora_a.untyped_data();
    p.lora_b = lora_b.untyped_data();
    p.lora_scaling = lora_scaling.typed_data();
    if (adapter_indices.element_count() > 0) {
      if (adapter_indices.element_count() != p.m)
        return ffi::Error::InvalidArgument("adapter_indices must hold one entry per row");
      p.adapter_indices = adapter_indices.typed_data();
    }
  }
  if (y->element_count() != static_cast<size_t>(p.m) * p.n) return ffi::Error::InvalidArgument("result must be bf16 [..., N]");
  p.x = x.untyped_data();
  p.w_packed = w_packed.untyped_data();
  p.w_scales = w_scales.typed_data();
  p.out = y->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  return ToError(mi355_w8a8_gq_linear_v1(&p, stream), "mi355_w8a8 gq linear launch submission failed");
}

// Backward of the grouped call (mi355_w8a8_grouped_bwd_v1).  x [M, K] and dy [M, N] bf16 in group order, packed
// weights, scales f32 [n_weights, N], A [G, K, r], B [G, r, N], scaling [G] (size-0 without LoRA), group_sizes
// s32 [G].  Results: dx bf16 [M, K], dA, dB bf16 like A, B, dscaling f32 [G] (size 0 without LoRA), workspace u8.
ffi::Error GroupedBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::BF16> dy,
                      ffi::Buffer<ffi::U8> w_packed, ffi::Buffer<ffi::F32> w_scales, ffi::Buffer<ffi::BF16> lora_a,
                      ffi::Buffer<ffi::BF16> lora_b, ffi::Buffer<ffi::F32> lora_scaling,
                      ffi::Buffer<ffi::S32> group_sizes, ffi::ResultBuffer<ffi::BF16> dx,
                      ffi::ResultBuffer<ffi::BF16> d_lora_a, ffi::ResultBuffer<ffi::BF16> d_lora_b,
                      ffi::ResultBuffer<ffi::F32> d_lora_scaling, ffi::ResultBuffer<ffi::U8> workspace) {
  mi355_w8a8_grouped_bwd_problem p{};
  p.struct_size = sizeof(p);
  if (!RowsAndK(x.dimensions(), &p.m, &p.k))
    return ffi::Error::InvalidArgument("x must be bf16 [M, K] with a non-empty row domain");
  auto ds = w_scales.dimensions();
  if (ds.size() != 2 || ds[0] <= 0 || ds[1] <= 0) return ffi::Error::InvalidArgument("w_scales must be f32 [n_weights, N]");
  const uint32_t n_weights = static_cast<uint32_t>(ds[0]);
  p.n = static_cast<uint32_t>(ds[1]);
  p.n_groups = static_cast<uint32_t>(group_sizes.element_count());
  if (p.n_groups == 0 || p.n_groups % n_weights != 0)
    return ffi::Error::InvalidArgument("group_sizes must be s32 [G] with G a multiple of the number of weights");
  p.groups_per_weight = p.n_groups / n_weights;
  if (dy.element_count() != static_cast<size_t>(p.m) * p.n || dx->element_count() != x.element_count())
    return ffi::Error::InvalidArgument("dy must be bf16 [M, N] and dx must match x");
  if (w_packed.size_bytes() != static_cast<size_t>(n_weights) * mi355_w8a8_packed_weight_bytes(p.k, p.n))
    return ffi::Error::InvalidArgument("packed weights do not match (n_weights, K, N)");
  if (lora_a.element_count() > 0) {
    auto da = lora_a.dimensions();
    auto db = lora_b.dimensions();
    if (da.size() != 3 || db.size() != 3 || da[0] != p.n_groups || da[1] != p.k || db[0] != da[0] ||
        db[1] != da[2] || db[2] != p.n || lora_scaling.element_count() != p.n_groups)
      return ffi::Error::InvalidArgument("LoRA A/B/scaling must be [G,K,r], [G,r,N], [G]");
    if (d_lora_a->element_count() != lora_a.element_count() || d_lora_b->element_count() != lora_b.element_count() ||
        d_lora_scaling->element_count() != lora_scaling.element_count())
      return ffi::Error::InvalidArgument("the LoRA cotangents must match the LoRA parameters");
    p.rank = static_cast<uint32_t>(da[2]);
    p.lora_a = lora_a.untyped_data();
    p.lora_b = lora_b.untyped_data();
    p.lora_scaling = lora_scaling.typed_data();
    p.d_lora_a = d_lora_a->untyped_data();
    p.d_lora_b = d_lora_b->untyped_data();
    p.d_lora_scaling = d_lora_scaling->typed_data();
  }
  p.x = x.untyped_data();
  p.dy = dy.untyped_data();
  p.w_packed = w_packed.untyped_data();
  p.w_scales = w_scales.typed_data();
  p.group_sizes = group_sizes.typed_data();
  p.dx = dx->untyped_data();
  p.workspace = workspace->untyped_data();
  p.workspace_bytes = workspace->size_bytes();
  return ToError(mi355_w8a8_grouped_bwd_v1(&p, stream), "mi355_w8a8 grouped backward launch submission failed");
}

// Pull-back of the attention input stage.  fused bf16 [M, width], the two head-norm weights f32 [D], positions
// s32 [M], the four output cotangents.  Results: d_fused bf16 [M, width], d_q_norm_weight and d_k_norm_weight
// f32 [D] (size 0: not wanted, both or neither), workspace u8 (size 0 without the weight cotangents).
ffi::Error QkvSplitNormRopeBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> fused, ffi::Buffer<ffi::F32> q_norm_weight,
                               ffi::Buffer<ffi::F32> k_norm_weight, ffi::Buffer<ffi::S32> positions,
                               ffi::Buffer<ffi::BF16> d_q, ffi::Buffer<ffi::BF16> d_k, ffi::Buffer<ffi::BF16> d_v,
                               ffi::Buffer<ffi::BF16> d_gate, ffi::ResultBuffer<ffi::BF16> d_fused,
                               ffi::ResultBuffer<ffi::F32> d_q_norm_weight, ffi::ResultBuffer<ffi::F32> d_k_norm_weight,
                               ffi::ResultBuffer<ffi::U8> workspace, int32_t rotary_dim, float rope_theta,
                               float rms_eps) {
  mi355_w8a8_qkv_post_bwd_problem p{};
  p.struct_size = sizeof(p);
  auto dq = d_q.dimensions();
  auto dk = d_k.dimensions();
  if (dq.size() != 3 || dk.size() != 3 || dq[0] <= 0 || dk[0] != dq[0] || dk[2] != dq[2] || dq[1] <= 0 || dk[1] <= 0)
    return ffi::Error::InvalidArgument("d_q must be bf16 [M, H, D] and d_k bf16 [M, Hkv, D]");
  p.m = static_cast<uint32_t>(dq[0]);
  p.num_query_heads = static_cast<uint32_t>(dq[1]);
  p.num_kv_heads = static_cast<uint32_t>(dk[1]);
  p.head_dim = static_cast<uint32_t>(dq[2]);
  const size_t width = static_cast<size_t>(p.num_query_heads) * 2 * p.head_dim + 2 * static_cast<size_t>(p.num_kv_heads) * p.head_dim;
  if (fused.element_count() != static_cast<size_t>(p.m) * width || d_fused->element_count() != fused.element_count() ||
      d_v.element_count() != d_k.element_count() || d_gate.element_count() != d_q.element_count() ||
      positions.element_count() != p.m || q_norm_weight.element_count() != p.head_dim ||
      k_norm_weight.element_count() != p.head_dim)
    return ffi::Error::InvalidArgument("fused, d_fused, d_v, d_gate, positions or the norm weights do not match (M, H, Hkv, D)");
  if (rotary_dim < 0) return ffi::Error::InvalidArgument("rotary_dim must be >= 0");
  const bool want_w = d_q_norm_weight->element_count() > 0 || d_k_norm_weight->element_count() > 0;
  if (want_w) {
    if (d_q_norm_weight->element_count() != p.head_dim || d_k_norm_weight->element_count() != p.head_dim)
      return ffi::Error::InvalidArgument("the norm-weight cotangents must both be f32 [D], or both empty");
    p.d_q_norm_weight = d_q_norm_weight->typed_data();
    p.d_k_norm_weight = d_k_norm_weight->typed_data();
    p.workspace = workspace->untyped_data();
    p.workspace_bytes = workspace->size_bytes();
  }
  p.rotary_dim = static_cast<uint32_t>(rotary_dim);
  p.rope_theta = rope_theta;
  p.rms_eps = rms_eps;
  p.fused = fused.untyped_data();
  p.q_norm_weight = q_norm_weight.typed_data();
  p.k_norm_weight = k_norm_weight.typed_data();
  p.positions = positions.typed_data();
  p.d_q = d_q.untyped_data();
  p.d_k = d_k.untyped_data();
  p.d_v = d_v.untyped_data();
  p.d_gate = d_gate.untyped_data();
  p.d_fused = d_fused->untyped_data();
  return ToError(mi355_w8a8_qkv_split_norm_rope_bwd_v1(&p, stream), "mi355_w8a8 qkv stage backward launch submission failed");
}

// Pull-back of the decoder norm in delta form: x, d_normalized bf16 [.., K], gamma f32 [K].  Results: d_x bf16
// [.., K], d_gamma f32 [K] (size 0: not wanted), workspace u8 (size 0 without d_gamma).
ffi::Error DeltaRmsNormBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::F32> gamma,
                           ffi::Buffer<ffi::BF16> d_normalized, ffi::ResultBuffer<ffi::BF16> d_x,
                           ffi::ResultBuffer<ffi::F32> d_gamma, ffi::ResultBuffer<ffi::U8> workspace, float eps) {
  uint32_t m = 0, k = 0;
  if (!RowsAndK(x.dimensions(), &m, &k))
    return ffi::Error::InvalidArgument("x must be bf16 [..., K] with a non-empty row domain");
  if (gamma.element_count() != k || d_normalized.element_count() != x.element_count() ||
      d_x->element_count() != x.element_count() || (d_gamma->element_count() != 0 && d_gamma->element_count() != k))
    return ffi::Error::InvalidArgument("gamma must be f32 [K]; d_normalized and d_x must match x; d_gamma f32 [K] or empty");
  const bool want_g = d_gamma->element_count() > 0;
  return ToError(mi355_w8a8_delta_rms_norm_bwd_v1(x.untyped_data(), gamma.typed_data(), d_normalized.untyped_data(),
                                                  d_x->untyped_data(), want_g ? d_gamma->typed_data() : nullptr,
                                                  want_g ? workspace->untyped_data() : nullptr,
                                                  want_g ? workspace->size_bytes() : 0, m, k, eps, stream),
                 "mi355_w8a8 delta rms norm pull-back launch submission failed");
}

// Pull-back of the router: logits f32 [T, E], selected s32 [T, top_k], d_weights f32 [T, top_k] -> d_logits f32 [T, E].
ffi::Error MoeRouteBwd(hipStream_t stream, ffi::Buffer<ffi::F32> router_logits, ffi::Buffer<ffi::S32> selected,
                       ffi::Buffer<ffi::F32> d_weights, ffi::ResultBuffer<ffi::F32> d_router_logits,
                       int32_t norm_topk_prob) {
  auto d = router_logits.dimensions();
  auto dw = d_weights.dimensions();
  if (d.size() != 2 || dw.size() != 2 || d[0] <= 0 || dw[0] != d[0] || dw[1] <= 0 ||
      selected.element_count() != d_weights.element_count() ||
      d_router_logits->element_count() != router_logits.element_count())
    return ffi::Error::InvalidArgument("router_logits and d_router_logits must be f32 [T, E]; selected and d_weights [T, top_k]");
  return ToError(mi355_w8a8_moe_route_bwd_v1(router_logits.typed_data(), selected.typed_data(), d_weights.typed_data(),
                                             static_cast<uint32_t>(d[0]), static_cast<uint32_t>(d[1]),
                                             static_cast<uint32_t>(dw[1]), norm_topk_prob ? 1u : 0u,
                                             d_router_logits->typed_data(), stream),
                 "mi355_w8a8 moe route pull-back launch submission failed");
}

// Pull-back of the combine: d_out bf16 [T, H], expert_out bf16 [T top_k, H] in sorted order, sort_indices s32
// [T top_k], weights f32 [T, top_k].  Results: d_expert_out bf16 [T top_k, H], d_weights f32 [T, top_k].
ffi::Error MoeCombineBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> d_out, ffi::Buffer<ffi::BF16> expert_out,
                         ffi::Buffer<ffi::S32> sort_indices, ffi::Buffer<ffi::F32> weights,
                         ffi::ResultBuffer<ffi::BF16> d_expert_out, ffi::ResultBuffer<ffi::F32> d_weights) {
  auto dd = d_out.dimensions();
  auto dw = weights.dimensions();
  if (dd.size() != 2 || dw.size() != 2 || dw[0] != dd[0] || dw[0] <= 0 || dw[1] <= 0 || dd[1] <= 0)
    return ffi::Error::InvalidArgument("d_out must be bf16 [T, H] and weights f32 [T, top_k]");
  const size_t pairs = static_cast<size_t>(dw[0]) * dw[1];
  if (expert_out.element_count() != pairs * dd[1] || d_expert_out->element_count() != pairs * dd[1] ||
      sort_indices.element_count() != pairs || d_weights->element_count() != pairs)
    return ffi::Error::InvalidArgument("expert_out and d_expert_out must be [T * top_k, H]; sort_indices and d_weights hold T * top_k entries");
  return ToError(mi355_w8a8_moe_combine_bwd_v1(d_out.untyped_data(), expert_out.untyped_data(), sort_indices.typed_data(),
                                               weights.typed_data(), d_expert_out->untyped_data(), d_weights->typed_data(),
                                               static_cast<uint32_t>(dw[0]), static_cast<uint32_t>(dw[1]),
                                               static_cast<uint32_t>(dd[1]), stream),
                 "mi355_w8a8 moe combine pull-back launch submission failed");
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_forward_v1, Forward,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("swiglu")
                                  .Attr<float>("rms_eps")
                                  .Attr<int32_t>("entry"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_quantize_rows_v1, QuantizeRows,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::S8>>()
                                  .Ret<ffi::Buffer<ffi::F32>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_pack_weight_v1, PackWeight,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::S8>>()
                                  .Ret<ffi::Buffer<ffi::U8>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_backward_v1, Backward,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>());
XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_swiglu_bwd_v1, SwigluBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_rms_norm_bwd_v1, RmsNormBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Attr<float>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_moe_route_v1, MoeRoute,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Attr<int32_t>("norm_topk_prob"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_moe_dispatch_v1, MoeDispatch,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("repeat"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_moe_combine_v1, MoeCombine,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>());
XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_grouped_v1, Grouped,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("swiglu")
                                  .Attr<int32_t>("x_row_repeat"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_qkv_split_norm_rope_v1, QkvSplitNormRope,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Attr<int32_t>("rotary_dim")
                                  .Attr<float>("rope_theta")
                                  .Attr<float>("rms_eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_gq_pack_weight_v1, GqPackWeight,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::S8>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("weight_bits"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_gq_linear_v1, GqLinear,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("group_size")
                                  .Attr<int32_t>("weight_bits")
                                  .Attr<int32_t>("activation_bits"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_grouped_bwd_v1, GroupedBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_qkv_split_norm_rope_bwd_v1, QkvSplitNormRopeBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<int32_t>("rotary_dim")
                                  .Attr<float>("rope_theta")
                                  .Attr<float>("rms_eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_delta_rms_norm_bwd_v1, DeltaRmsNormBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<float>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_moe_route_bwd_v1, MoeRouteBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Attr<int32_t>("norm_topk_prob"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(mi355_w8a8_ffi_moe_combine_bwd_v1, MoeCombineBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>());
#endif  // __has_include("xla/ffi/api/ffi.h")
