// Flattens the C++ LowOHA arguments (std::vector, std::string, nested structs)
// into the plain structs of the C ABI and forwards the call.  The caller's
// objects are read, never modified (reorder_params_t::prepack.cached_size aside,
// as in the reference).
#include "zendnnl_lowoha.hpp"

#include <algorithm>

#include "zmi_lowoha.h"

namespace zendnnl {
namespace lowoha {

namespace {
template <typename Q>
zmi_quant_t flat_quant(const Q &q) {
  zmi_quant_t f{};
  f.buff = q.buff;
  f.dt = static_cast<int32_t>(q.dt);
  f.ndims = static_cast<int32_t>(std::min<size_t>(q.dims.size(), ZMI_MAX_DIMS));
  for (int i = 0; i < f.ndims; ++i) f.dims[i] = q.dims[i];
  return f;
}

// Owns the post-op array a flattened matmul_params points at.
struct FlatParams {
  zmi_matmul_params_t p;
  std::vector<zmi_post_op_t> po;
};

void flatten(const matmul::matmul_params &s, FlatParams &out) {
  zmi_matmul_params_t &p = out.p;
  zmi_matmul_params_init(&p);
  p.dt_src = static_cast<int32_t>(s.dtypes.src);
  p.dt_wei = static_cast<int32_t>(s.dtypes.wei);
  p.dt_dst = static_cast<int32_t>(s.dtypes.dst);
  p.dt_bias = static_cast<int32_t>(s.dtypes.bias);
  p.dt_compute = static_cast<int32_t>(s.dtypes.compute);
  out.po.resize(s.postop_.size());
  for (size_t i = 0; i < s.postop_.size(); ++i) {
    const matmul::matmul_post_op &a = s.postop_[i];
    zmi_post_op_t &b = out.po[i];
    b = zmi_post_op_t{};
    b.po_type = static_cast<int32_t>(a.po_type);
    b.dtype = static_cast<int32_t>(a.dtype);
    b.buff = a.buff;
    b.ndims = static_cast<int32_t>(std::min<size_t>(a.dims.size(), ZMI_MAX_DIMS));
    for (int d = 0; d < b.ndims; ++d) b.dims[d] = a.dims[d];
    b.leading_dim = a.leading_dim;
    b.alpha = a.alpha;
    b.beta = a.beta;
  }
  p.n_postops = static_cast<int32_t>(out.po.size());
  p.postops = out.po.empty() ? nullptr : out.po.data();
  p.src_scale = flat_quant(s.quant_params.src_scale);
  p.wei_scale = flat_quant(s.quant_params.wei_scale);
  p.dst_scale = flat_quant(s.quant_params.dst_scale);
  p.src_zp = flat_quant(s.quant_params.src_zp);
  p.wei_zp = flat_quant(s.quant_params.wei_zp);
  p.dst_zp = flat_quant(s.quant_params.dst_zp);
  p.mem_format_a = s.mem_format_a;
  p.mem_format_b = s.mem_format_b;
  p.lowoha_algo = static_cast<int32_t>(s.lowoha_algo);
  p.num_threads = s.num_threads;
  p.dynamic_quant = s.dynamic_quant ? 1 : 0;
  p.pack_format_b = s.packing.pack_format_b;
  p.total_matmul = s.total_matmul;
  p.active_matmul = s.active_matmul;
  p.weight_cache_type = s.weight_cache_type;
}

std::vector<uint8_t> bytes_of(const std::vector<bool> &v) {
  std::vector<uint8_t> o(v.size());
  for (size_t i = 0; i < v.size(); ++i) o[i] = v[i] ? 1 : 0;
  return o;
}

zmi_reorder_params_t flatten(const reorder::reorder_params_t &s) {
  zmi_reorder_params_t r;
  zmi_reorder_params_init(&r);
  r.src_dtype = static_cast<int32_t>(s.src_dtype);
  r.dst_dtype = static_cast<int32_t>(s.dst_dtype);
  r.scale = flat_quant(s.quant_params.scale);
  r.zero_point = flat_quant(s.quant_params.zero_point);
  r.algo = static_cast<int32_t>(s.algo);
  r.num_threads = s.num_threads;
  auto put = [](const std::vector<int64_t> &v, int32_t &n, int64_t *dst) {
    n = static_cast<int32_t>(std::min<size_t>(v.size(), ZMI_MAX_DIMS));
    for (int i = 0; i < n; ++i) dst[i] = v[i];
  };
  put(s.src_shape, r.n_src_shape, r.src_shape);
  put(s.dst_shape, r.n_dst_shape, r.dst_shape);
  put(s.src_strides, r.n_src_strides, r.src_strides);
  put(s.dst_strides, r.n_dst_strides, r.dst_strides);
  r.dynamic_quant = s.dynamic_quant ? 1 : 0;
  r.is_prepack = s.is_prepack ? 1 : 0;
  r.prepack.algo = static_cast<int32_t>(s.prepack.algo);
  r.prepack.wei_dtype = static_cast<int32_t>(s.prepack.wei_dtype);
  r.prepack.src_dtype = static_cast<int32_t>(s.prepack.src_dtype);
  r.prepack.K = s.prepack.K;
  r.prepack.N = s.prepack.N;
  r.prepack.ldb = s.prepack.ldb;
  r.prepack.transposed = s.prepack.transposed ? 1 : 0;
  r.prepack.sym_group_size = s.prepack.sym_group_size;
  r.prepack.cached_size = s.prepack.cached_size;
  return r;
}
}  // namespace

namespace matmul {

status_t matmul_direct(const char layout, const bool transA, const bool transB, const int M, const int N,
                       const int K, const float alpha, const void *src, const int lda, const void *weight,
                       const int ldb, const void *bias, const float beta, void *dst, const int ldc,
                       const bool is_weights_const, const matmul_batch_params_t &batch_params,
                       const matmul_params &params) {
  FlatParams fp;
  flatten(params, fp);
  zmi_batch_params_t b;
  b.Batch_A = batch_params.Batch_A;
  b.Batch_B = batch_params.Batch_B;
  b.batch_stride_src = batch_params.batch_stride_src;
  b.batch_stride_wei = batch_params.batch_stride_wei;
  b.batch_stride_dst = batch_params.batch_stride_dst;
  return static_cast<status_t>(zmi_matmul_direct(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb,
                                                 bias, beta, dst, ldc, is_weights_const, &b, &fp.p));
}

status_t group_matmul_direct(const std::vector<char> &layout, const std::vector<bool> &transA,
                             const std::vector<bool> &transB, const std::vector<int> &M,
                             const std::vector<int> &N, const std::vector<int> &K,
                             const std::vector<float> &alpha, const std::vector<const void *> &src,
                             const std::vector<int> &lda, const std::vector<const void *> &weight,
                             const std::vector<int> &ldb, const std::vector<const void *> &bias,
                             const std::vector<float> &beta, const std::vector<void *> &dst,
                             const std::vector<int> &ldc, const std::vector<bool> &is_weights_const,
                             const std::vector<matmul_params> &params,
                             const group_matmul_moe_postop_params *moe_postop,
                             const grp_matmul_gated_act_params *gated_act,
                             const grp_matmul_fused_moe_params *fused_moe) {
  const std::vector<uint8_t> ta = bytes_of(transA), tb = bytes_of(transB), wc = bytes_of(is_weights_const);
  std::vector<FlatParams> fps(params.size());
  std::vector<zmi_matmul_params_t> fp(params.size());
  for (size_t i = 0; i < params.size(); ++i) {
    flatten(params[i], fps[i]);
    fp[i] = fps[i].p;
  }
  zmi_group_args_t g{};
  auto n = [](size_t s) { return static_cast<int32_t>(s); };
  g.n_layout = n(layout.size()); g.layout = layout.data();
  g.n_transA = n(ta.size()); g.transA = ta.data();
  g.n_transB = n(tb.size()); g.transB = tb.data();
  g.n_M = n(M.size()); g.M = M.data();
  g.n_N = n(N.size()); g.N = N.data();
  g.n_K = n(K.size()); g.K = K.data();
  g.n_alpha = n(alpha.size()); g.alpha = alpha.data();
  g.n_src = n(src.size()); g.src = src.data();
  g.n_lda = n(lda.size()); g.lda = lda.data();
  g.n_weight = n(weight.size()); g.weight = weight.data();
  g.n_ldb = n(ldb.size()); g.ldb = ldb.data();
  g.n_bias = n(bias.size()); g.bias = bias.data();
  g.n_beta = n(beta.size()); g.beta = beta.data();
  g.n_dst = n(dst.size()); g.dst = dst.data();
  g.n_ldc = n(ldc.size()); g.ldc = ldc.data();
  g.n_is_weights_const = n(wc.size()); g.is_weights_const = wc.data();
  g.n_params = n(fp.size()); g.params = fp.data();

  zmi_moe_postop_t pp{};
  if (moe_postop) {
    pp.num_tokens = moe_postop->num_tokens;
    pp.topk = moe_postop->topk;
    pp.output = moe_postop->output;
    pp.ldc_output = moe_postop->ldc_output;
    pp.topk_weights = moe_postop->topk_weights;
    pp.skip_weighted = moe_postop->skip_weighted ? 1 : 0;
    pp.row_ptrs = moe_postop->row_ptrs;
  }
  zmi_fused_moe_t fm{};
  std::vector<zmi_quant_t> dscale, dzp;
  if (fused_moe) {
    const grp_matmul_fused_moe_params &f = *fused_moe;
    fm.n_down_weight = n(f.down_weight.size()); fm.down_weight = f.down_weight.data();
    fm.n_N_down = n(f.N_down.size()); fm.N_down = f.N_down.data();
    fm.n_ldb_down = n(f.ldb_down.size()); fm.ldb_down = f.ldb_down.data();
    fm.n_bias_down = n(f.bias_down.size()); fm.bias_down = f.bias_down.data();
    fm.bias_dt_down = static_cast<int32_t>(f.bias_dt_down);
    for (const auto &q : f.down_scale) dscale.push_back(flat_quant(q));
    for (const auto &q : f.down_zp) dzp.push_back(flat_quant(q));
    fm.n_down_scale = n(dscale.size()); fm.down_scale = dscale.data();
    fm.n_down_zp = n(dzp.size()); fm.down_zp = dzp.data();
    fm.n_dst_down = n(f.dst_down.size()); fm.dst_down = f.dst_down.data();
    fm.n_ldc_down = n(f.ldc_down.size()); fm.ldc_down = f.ldc_down.data();
  }
  return static_cast<status_t>(zmi_group_matmul_direct(&g, moe_postop ? &pp : nullptr,
                                                       gated_act ? static_cast<int32_t>(gated_act->act) : 0,
                                                       fused_moe ? &fm : nullptr));
}

void clear_matmul_weight_caches() { zmi_clear_weight_cache(); }
void clear_fused_moe_scratch() { zmi_clear_scratch(); }

}  // namespace matmul

namespace reorder {

status_t reorder_direct(const void *src, void *dst, reorder_params_t &params) {
  zmi_reorder_params_t r = flatten(params);
  return static_cast<status_t>(zmi_reorder_direct(src, dst, &r));
}

size_t weight_prepack_size(const reorder_params_t &params) {
  zmi_reorder_params_t r = flatten(params);
  const size_t s = zmi_weight_prepack_size(&r);
  params.prepack.cached_size = r.prepack.cached_size;
  return s;
}

status_t group_dynamic_quant(const std::vector<const void *> &src, const std::vector<int> &M,
                             const std::vector<int> &K, const std::vector<std::vector<int64_t>> &src_strides,
                             const std::vector<void *> &dst, const std::vector<std::vector<int64_t>> &dst_strides,
                             const std::vector<void *> &scale, const group_dynamic_quant_params_t &params) {
  const size_t n = src.size();
  if (M.size() != n || K.size() != n || dst.size() != n || scale.size() != n ||
      (!src_strides.empty() && src_strides.size() != n) || (!dst_strides.empty() && dst_strides.size() != n))
    return status_t::failure;
  std::vector<int64_t> ss(n, 0), ds(n, 0);
  for (size_t i = 0; i < n; ++i) {
    if (!src_strides.empty() && !src_strides[i].empty()) {
      if (src_strides[i].size() != 2 || src_strides[i][1] != 1) return status_t::failure;
      ss[i] = src_strides[i][0];
    }
    if (!dst_strides.empty() && !dst_strides[i].empty()) {
      if (dst_strides[i].size() != 2 || dst_strides[i][1] != 1) return status_t::failure;
      ds[i] = dst_strides[i][0];
    }
  }
  zmi_group_dq_params_t p;
  p.src_dtype = static_cast<int32_t>(params.src_dtype);
  p.dst_dtype = static_cast<int32_t>(params.dst_dtype);
  p.scale_dtype = static_cast<int32_t>(params.scale_dtype);
  p.num_threads = params.num_threads;
  p.num_groups = params.num_groups;
  return static_cast<status_t>(zmi_group_dynamic_quant(static_cast<int32_t>(n), src.data(), M.data(), K.data(),
                                                       ss.data(), dst.data(), ds.data(), scale.data(), &p));
}

}  // namespace reorder
}  // namespace lowoha
}  // namespace zendnnl
