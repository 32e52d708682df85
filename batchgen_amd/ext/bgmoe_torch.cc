// PyTorch-ROCm C++ extension modules over libbgmoe.so's C ABI, under the reference's module and op names:
//   batchgen_kernels.moe._C_routing                    (batchgen_kernels/src/moe/routing/routing_extension.cc:11-137)
//   batchgen_kernels.common._C_mgn_ops                 (batchgen_kernels/src/moe/mgn/mgn_extension.cc:17-62)
//   batchgen_kernels.moe._C_dispatch_scatter_3d        (batchgen_kernels/src/moe/dispatch_scatter_3d.cu:671-683)
//   batchgen_kernels.moe._C_fp8_blockwise_gemm         (batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_gemm.cu:1253-1299)
//   batchgen_kernels.moe._C_fp8_blockwise_ops          (batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_ops.cu:800-814)
//   batchgen_kernels.attention._C_add_rmsnorm_fp8_quant (batchgen_kernels/src/attention/csrc/add_rmsnorm_fp8_quant.cu:553-566)
// One translation unit defines every module's PyInit function; the build installs the one shared object under each
// module's file name.  An op checks its tensors (device, dtype, shape, contiguity: TORCH_CHECK, i.e. RuntimeError,
// as the reference's bindings), allocates what the reference op allocates, and enqueues on the current stream.
// Host code only: the kernels live in libbgmoe.so.  (PyTorch-ROCm calls its device type "cuda": the guard and the
// stream are the ...MasqueradingAsCUDA ones.)
#include <torch/python.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/bgmoe.h"

namespace {

using torch::Tensor;
using OptTensor = c10::optional<Tensor>;

void check_rc(int rc) {
  TORCH_CHECK(rc == BGMOE_OK, bgmoe_last_error());
}
bgmoe_stream_t cur_stream() { return reinterpret_cast<bgmoe_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()); }
bool given(const OptTensor& t) { return t.has_value() && t->defined() && t->numel() > 0; }
bool fp8_bytes(const Tensor& t) { return t.scalar_type() == at::kByte || t.scalar_type() == at::kFloat8_e4m3fn; }

void want(const Tensor& t, const char* name, c10::optional<at::ScalarType> dt = c10::nullopt) {
  TORCH_CHECK(t.defined() && t.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  if (dt.has_value()) TORCH_CHECK(t.scalar_type() == *dt, name, " must be ", *dt, ", got ", t.scalar_type());
}
void same_device(const Tensor& ref, const Tensor& t, const char* name) {
  TORCH_CHECK(t.device() == ref.device(), name, " must be on ", ref.device());
}
template <typename T = void>
T* ptr(const Tensor& t) { return t.defined() ? reinterpret_cast<T*>(t.data_ptr()) : nullptr; }
template <typename T = void>
T* optr(const OptTensor& t) { return given(t) ? reinterpret_cast<T*>(t->data_ptr()) : nullptr; }

// Scratch for ops whose reference signature carries no workspace: one buffer per (kind, device, stream), never freed
// once handed out (a captured graph keeps writing to it), growth doubles.
Tensor scratch(int kind, const at::Device& dev, size_t need, size_t floor) {
  static std::mutex mu;
  static std::map<std::tuple<int, int, void*>, Tensor> live;
  static std::vector<Tensor> retired;
  std::lock_guard<std::mutex> lock(mu);
  const auto key = std::make_tuple(kind, (int)dev.index(), (void*)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).stream());
  auto it = live.find(key);
  if (it == live.end() || (size_t)it->second.numel() < need) {
    size_t size = std::max(need, floor);
    if (it != live.end()) {
      size = std::max(size, 2 * (size_t)it->second.numel());
      retired.push_back(it->second);
    }
    live[key] = torch::empty({(int64_t)size}, torch::TensorOptions().dtype(at::kByte).device(dev));
    it = live.find(key);
  }
  return it->second;
}
Tensor dispatch_ws(const at::Device& dev, int64_t nk, int e_local) {
  const size_t need = bgmoe_dispatch_workspace_bytes(nk, e_local);
  return need ? scratch(0, dev, need, 1 << 20) : Tensor();
}

// ------------------------------------------------------------------------------------------- _C_routing
std::vector<Tensor> gate_impl(Tensor logits, Tensor bias, int64_t k, double rsf, Tensor ids, Tensor w, OptTensor num_valid,
                              OptTensor latent_out, int64_t latent_offset, OptTensor rank_counts, int64_t rows_per_rank,
                              int64_t max_e, bool allow_i64) {
  TORCH_CHECK(logits.defined() && logits.is_cuda(), "router_logits must be a CUDA tensor");
  TORCH_CHECK(logits.scalar_type() == at::kFloat, "router_logits must be FP32");
  TORCH_CHECK(logits.dim() == 2 && logits.stride(1) == 1, "router_logits must be 2-D with contiguous rows");
  want(bias, "e_score_correction", at::kFloat);
  const int64_t n = logits.size(0), e = logits.size(1);
  TORCH_CHECK(e <= max_e, "E=", e, " exceeds MAX_EXPERTS=", max_e);
  TORCH_CHECK(e >= k, "E=", e, " must be at least k=", k);
  TORCH_CHECK(bias.numel() == e, "e_score_correction must have E elements");
  if (!ids.defined() || ids.numel() == 0) ids = torch::empty({n, k}, logits.options().dtype(at::kInt));
  if (!w.defined() || w.numel() == 0) w = torch::empty({n, k}, logits.options());
  want(ids, "topk_indices");
  TORCH_CHECK(ids.scalar_type() == at::kInt || (allow_i64 && ids.scalar_type() == at::kLong), "topk_indices must be int32",
              allow_i64 ? " or int64" : "");
  want(w, "topk_weights", at::kFloat);
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == n && ids.size(1) == k && w.dim() == 2 && w.size(0) == n && w.size(1) == k,
              "topk_indices / topk_weights must be contiguous [", n, ", ", k, "] tensors");
  const int32_t* nv = nullptr;
  const int64_t* rc = nullptr;
  int rpr = 0;
  if (given(num_valid)) {
    TORCH_CHECK(!given(rank_counts), "num_valid_tokens and rank_token_counts are mutually exclusive");
    want(*num_valid, "num_valid_tokens", at::kInt);
    TORCH_CHECK(num_valid->numel() == 1, "num_valid_tokens must hold one int32");
    nv = ptr<int32_t>(*num_valid);
  } else if (given(rank_counts)) {
    want(*rank_counts, "rank_token_counts", at::kLong);
    rpr = (int)rows_per_rank;
    TORCH_CHECK(rpr > 0, "rows_per_rank must be positive when rank_token_counts is given");
    TORCH_CHECK(rank_counts->numel() * rpr == n, "rank_token_counts x rows_per_rank must equal N=", n);
    rc = ptr<int64_t>(*rank_counts);
  }
  uint16_t* lat = nullptr;
  int lat_off = 0, lat_size = 0;
  if (given(latent_out)) {
    want(*latent_out, "latent_out", at::kBFloat16);
    TORCH_CHECK(latent_out->dim() == 2 && latent_out->size(0) == n, "latent_out must have ", n, " rows");
    lat = ptr<uint16_t>(*latent_out);
    lat_off = (int)latent_offset;
    lat_size = (int)latent_out->size(1);
  }
  if (n == 0) return {ids, w};
  c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
  check_rc(bgmoe_gate_sigmoid_topk(ptr<float>(logits), logits.stride(0), ptr<float>(bias), (int)n, (int)e, (int)k, (float)rsf,
                                   ids.data_ptr(), ids.scalar_type() == at::kLong, ptr<float>(w), nv, rc, rpr, lat, lat_off,
                                   lat_size, cur_stream()));
  return {ids, w};
}

Tensor glm5_router_gemm(Tensor hidden, Tensor weight, OptTensor rank_counts, OptTensor output, int64_t bucket_size,
                        int64_t world_size) {
  want(hidden, "hidden_states", at::kBFloat16);
  want(weight, "router_weight", at::kBFloat16);
  same_device(hidden, weight, "router_weight");
  TORCH_CHECK(hidden.dim() == 2 && weight.dim() == 2 && hidden.size(1) == weight.size(1), "hidden_states [N,H] and "
              "router_weight [E,H] must share H");
  const int64_t n = hidden.size(0), h = hidden.size(1), e = weight.size(0);
  Tensor out = given(output) ? *output : torch::empty({n, e}, hidden.options().dtype(at::kFloat));
  want(out, "output", at::kFloat);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == n && out.size(1) == e, "output must be FP32 [", n, ", ", e, "]");
  const int64_t* rc = nullptr;
  if (given(rank_counts)) {
    want(*rank_counts, "rank_token_counts", at::kLong);
    TORCH_CHECK(rank_counts->numel() >= world_size, "rank_token_counts is shorter than world_size");
    TORCH_CHECK(bucket_size > 0, "bucket_size must be positive when rank_token_counts is provided");
    rc = ptr<int64_t>(*rank_counts);
  }
  if (n == 0 || e == 0) return out;
  c10::hip::HIPGuardMasqueradingAsCUDA guard(hidden.device());
  const size_t need = bgmoe_router_gemm_workspace_bytes((int)n, (int)h, (int)e);
  Tensor ws = need ? scratch(1, hidden.device(), need, 1 << 20) : Tensor();
  check_rc(bgmoe_router_gemm(ptr<uint16_t>(hidden), ptr<uint16_t>(weight), (int)n, (int)h, (int)e, rc, (int)bucket_size,
                             (int)world_size, ptr<float>(out), ptr(ws), ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  return out;
}

std::vector<Tensor> dispatch_count_gather(Tensor x, Tensor ids, int64_t expert_start, int64_t el, Tensor counts, Tensor offsets,
                                          Tensor counters, Tensor dispatched, Tensor pos, OptTensor rank_counts,
                                          c10::optional<int64_t> rows_per_rank) {
  TORCH_CHECK(!given(rank_counts), "dispatch_count_gather: rank_token_counts is not supported on one GPU");
  (void)rows_per_rank;
  want(x, "x", at::kBFloat16);
  want(ids, "topk_indices", at::kInt);
  for (auto* t : {&counts, &offsets, &counters, &pos}) want(*t, "index tensor", at::kInt);
  want(dispatched, "dispatched_x", at::kBFloat16);
  TORCH_CHECK(x.dim() == 2 && ids.dim() == 2 && ids.size(0) == x.size(0), "x [N,H] and topk_indices [N,K] mismatch");
  const int64_t n = x.size(0), h = x.size(1), k = ids.size(1);
  TORCH_CHECK(counts.numel() >= el && counters.numel() >= el && offsets.numel() >= el + 1 && pos.numel() >= n * k,
              "expert_counts / expert_counters [E], expert_offsets [E+1] or topk_pos [N*K] too small");
  TORCH_CHECK(dispatched.dim() == 2 && dispatched.size(1) == h, "dispatched_x must be BF16 [rows, H=", h, "]");
  for (auto* t : {&ids, &counts, &offsets, &counters, &dispatched, &pos}) same_device(x, *t, "every tensor");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor ws = dispatch_ws(x.device(), n * k, (int)el);
  check_rc(bgmoe_dispatch_scatter_ragged(ptr<uint16_t>(x), ptr<int32_t>(ids), (int)n, (int)k, (int)h, ptr<uint16_t>(dispatched),
                                         dispatched.size(0), (int)expert_start, (int)el, ptr<int32_t>(counts),
                                         ptr<int32_t>(counters), ptr<int32_t>(pos), ptr<int32_t>(offsets), 1, ptr(ws),
                                         ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  return {counts, offsets, pos};
}

Tensor combine(Tensor y, Tensor pos, Tensor w, int64_t N, int64_t H, int64_t K, Tensor out, int64_t num_valid) {
  TORCH_CHECK(K == 2 || K == 4 || K == 8, "Unsupported K=", K);
  want(y, "expert_output", at::kBFloat16);
  want(pos, "topk_pos", at::kInt);
  want(w, "topk_weights", at::kFloat);
  if (!out.defined() || out.numel() == 0) out = torch::zeros({N, H}, y.options());
  want(out, "output", at::kBFloat16);
  TORCH_CHECK(N >= 0 && H > 0, "N must be non-negative and H positive");
  // [rows, H] or the masked buffer [E_local, max_tokens, H]: topk_pos indexes rows of H elements either way
  TORCH_CHECK(y.dim() >= 2 && y.size(-1) == H, "expert_output must have rows of H=", H, " elements");
  TORCH_CHECK(pos.numel() >= N * K && w.numel() >= N * K && out.numel() >= N * H, "topk_pos / topk_weights / output too small");
  for (auto* t : {&pos, &w, &out}) same_device(y, *t, "topk_pos / topk_weights / output");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  check_rc(bgmoe_reduce_weighted_scatter(ptr<uint16_t>(y), ptr<int32_t>(pos), ptr<float>(w), (int)N, (int)H, (int)K,
                                         ptr<uint16_t>(out), (int)num_valid, nullptr, 0, cur_stream()));
  return out;
}

// ------------------------------------------------------------------------------------------- _C_mgn_ops
std::vector<Tensor> moe_fused_gate(Tensor scores, Tensor bias, int64_t n_group, int64_t topk_group, int64_t e, int64_t top_k,
                                   double rsf) {
  TORCH_CHECK(scores.is_cuda(), "scores must be a CUDA tensor");
  TORCH_CHECK(scores.dim() == 2 && scores.size(1) == e, "scores dimension 1 must match n_routed_experts (", e, ")");
  TORCH_CHECK(bias.numel() == e, "e_score_correction_bias size must match n_routed_experts (", e, ")");
  TORCH_CHECK(e % n_group == 0, "n_routed_experts (", e, ") must be divisible by n_group (", n_group, ")");
  scores = scores.contiguous().to(at::kFloat);
  bias = bias.to(scores.device()).contiguous().to(at::kFloat);
  const int64_t n = scores.size(0);
  Tensor ids = torch::empty({n, top_k}, scores.options().dtype(at::kInt));
  Tensor w = torch::empty({n, top_k}, scores.options());
  c10::hip::HIPGuardMasqueradingAsCUDA guard(scores.device());
  check_rc(bgmoe_fused_gate(ptr<float>(scores), ptr<float>(bias), (int)n, (int)e, (int)n_group, (int)topk_group, (int)top_k,
                            (float)rsf, 0, ptr<int32_t>(ids), ptr<float>(w), cur_stream()));
  return {ids, w};
}

std::vector<Tensor> compact_expert_data(Tensor counts) {
  want(counts, "expert_counts", at::kInt);
  const int64_t e = counts.numel();
  auto opt = counts.options();
  Tensor idx = torch::empty({e}, opt), size = torch::empty({e}, opt), start = torch::empty({e}, opt);
  Tensor num = torch::zeros({1}, opt);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(counts.device());
  check_rc(bgmoe_compact_expert_data(ptr<int32_t>(counts), (int)e, ptr<int32_t>(size), ptr<int32_t>(idx), ptr<int32_t>(start),
                                     ptr<int32_t>(num), cur_stream()));
  return {size, idx, start, num};
}

std::vector<Tensor> expert_bincount(Tensor eids, int64_t start, int64_t per_rank, torch::Device device) {
  (void)device;
  TORCH_CHECK(eids.is_cuda(), "eids must be a CUDA tensor");
  TORCH_CHECK(eids.scalar_type() == at::kInt, "eids must be int32");
  TORCH_CHECK(eids.dim() == 1, "eids must be 1-dimensional");
  eids = eids.contiguous();
  const int64_t n = eids.numel();
  auto opt = eids.options();
  Tensor counts = torch::empty({per_rank}, opt), counters = torch::empty({per_rank}, opt);
  Tensor pos = torch::empty({std::max<int64_t>(n, 1)}, opt), cu = torch::empty({per_rank + 1}, opt);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(eids.device());
  Tensor ws = dispatch_ws(eids.device(), n, (int)per_rank);
  check_rc(bgmoe_dispatch_scatter_ragged(nullptr, ptr<int32_t>(eids), (int)n, 1, 0, nullptr, 0, (int)start, (int)per_rank,
                                         ptr<int32_t>(counts), ptr<int32_t>(counters), ptr<int32_t>(pos), ptr<int32_t>(cu), 1,
                                         ptr(ws), ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  return compact_expert_data(counts);
}

std::vector<Tensor> fused_moe_token_dispatch(Tensor x, Tensor ids, Tensor token_idx, Tensor topk_pos_in, int64_t start,
                                             int64_t end) {
  (void)token_idx; (void)topk_pos_in;          // the reference's kernel ignores them too (fused_moe_token_dispatch.cu:59-88)
  TORCH_CHECK(x.is_cuda(), "global_x must be a CUDA tensor");
  TORCH_CHECK(ids.is_cuda(), "topk_idx must be a CUDA tensor");
  TORCH_CHECK(x.is_contiguous(), "global_x must be contiguous");
  TORCH_CHECK(ids.is_contiguous(), "topk_idx must be contiguous");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16, "global_x must be BF16");
  TORCH_CHECK(end > start, "routed_expert_end_idx must exceed routed_expert_start_idx");
  TORCH_CHECK(x.dim() == 2 && ids.dim() == 2 && ids.size(0) == x.size(0), "global_x [N, H] and topk_idx [N, K] must agree in N");
  same_device(x, ids, "topk_idx");
  const int64_t n = x.size(0), h = x.size(1), k = ids.size(1), el = end - start, nk = n * k;
  Tensor ids32 = ids.to(at::kInt).contiguous();
  auto iopt = ids32.options();
  const int64_t rows = std::max<int64_t>(nk, 1);
  Tensor out_x = torch::empty({rows, h}, x.options());
  Tensor counts = torch::empty({el}, iopt), counters = torch::empty({el}, iopt), pos = torch::empty({rows}, iopt);
  Tensor offsets = torch::empty({el + 1}, iopt);
  Tensor eids = torch::empty({rows}, iopt), toks = torch::empty({rows}, iopt), slots = torch::empty({rows}, iopt);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor ws = dispatch_ws(x.device(), nk, (int)el);
  check_rc(bgmoe_dispatch_scatter_ragged(ptr<uint16_t>(x), ptr<int32_t>(ids32), (int)n, (int)k, (int)h, ptr<uint16_t>(out_x), rows,
                                         (int)start, (int)el, ptr<int32_t>(counts), ptr<int32_t>(counters), ptr<int32_t>(pos),
                                         ptr<int32_t>(offsets), 1, ptr(ws), ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  check_rc(bgmoe_dispatch_row_metadata(ptr<int32_t>(ids32), ptr<int32_t>(pos), nk, (int)k, ptr<int32_t>(offsets) + el, rows,
                                       ptr<int32_t>(eids), ptr<int32_t>(toks), ptr<int32_t>(slots), cur_stream()));
  return {out_x, eids, toks, slots, counts, offsets};
}

// ------------------------------------------------------------------------------- _C_dispatch_scatter_3d
std::vector<Tensor> dispatch_scatter_3d(Tensor x, Tensor ids, Tensor act, int64_t expert_start, int64_t el, int64_t mtp,
                                        Tensor counts, Tensor counters, Tensor pos) {
  want(x, "x", at::kBFloat16);
  TORCH_CHECK(x.dim() == 2 && ids.dim() == 2, "x must be [N, H] and topk_indices [N, K]");
  TORCH_CHECK(ids.size(0) == x.size(0), "topk_indices has ", ids.size(0), " rows, x has ", x.size(0));
  const int64_t n = x.size(0), h = x.size(1), k = ids.size(1);
  Tensor flat = ids.reshape({-1}).contiguous();
  want(flat, "topk_indices", at::kInt);
  want(act, "act_buffer", at::kBFloat16);
  TORCH_CHECK(act.numel() >= el * mtp * h, "act_buffer is smaller than [E_local * max_tokens_padded, H]");
  for (auto* t : {&counts, &counters, &pos}) want(*t, "index tensor", at::kInt);
  TORCH_CHECK(counts.numel() >= el && counters.numel() >= el, "expert_counts / expert_counters must have E_local elements");
  TORCH_CHECK(pos.numel() >= n * k, "topk_pos must have N*K elements");
  for (auto* t : {&flat, &act, &counts, &counters, &pos}) same_device(x, *t, "every tensor");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor ws = dispatch_ws(x.device(), n * k, (int)el);
  check_rc(bgmoe_dispatch_scatter_3d(ptr<uint16_t>(x), ptr<int32_t>(flat), (int)n, (int)k, (int)h, ptr<uint16_t>(act),
                                     (int)expert_start, (int)el, (int)mtp, ptr<int32_t>(counts), ptr<int32_t>(counters),
                                     ptr<int32_t>(pos), ptr(ws), ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  return {counts, pos};
}

std::vector<Tensor> dispatch_scatter_ragged(Tensor x, Tensor ids, Tensor act, int64_t expert_start, int64_t el, Tensor counts,
                                            Tensor counters, Tensor pos, Tensor cu, int64_t row_align) {
  TORCH_CHECK(row_align > 0 && (row_align & (row_align - 1)) == 0 && row_align <= INT32_MAX,
              "row_align must be a positive power of two, got ", row_align);
  want(x, "x", at::kBFloat16);
  want(ids, "topk_indices", at::kInt);
  want(act, "act_buffer", at::kBFloat16);
  TORCH_CHECK(x.dim() == 2, "x must be BF16 [N, H]");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == x.size(0), "topk_indices must be int32 [N, K]");
  TORCH_CHECK(act.dim() == 2 && act.size(1) == x.size(1), "act_buffer must be BF16 [rows, H]");
  const int64_t n = x.size(0), h = x.size(1), k = ids.size(1), nk = n * k;
  TORCH_CHECK(expert_start >= 0 && expert_start + el <= INT32_MAX, "expert_start out of range: ", expert_start);
  const int64_t cap = (nk + (row_align - 1) * std::min(el, nk)) / row_align * row_align;
  TORCH_CHECK(cap <= act.size(0) && act.size(0) <= INT32_MAX, "act_buffer rows (", act.size(0), ") must be in [", cap,
              ", INT32_MAX]");
  for (auto* t : {&counts, &counters, &pos, &cu}) want(*t, "index tensor", at::kInt);
  TORCH_CHECK(counts.dim() == 1 && counts.size(0) == el, "expert_counts must be int32 [E_local]");
  TORCH_CHECK(counters.dim() == 1 && counters.size(0) == el, "expert_counters must be int32 [E_local]");
  TORCH_CHECK(cu.dim() == 1 && cu.size(0) == el + 1, "cu_seqlens must be int32 [E_local + 1]");
  TORCH_CHECK(pos.dim() == 1 && pos.size(0) == nk, "topk_pos must be int32 [N * K]");
  for (auto* t : {&ids, &act, &counts, &counters, &pos, &cu}) same_device(x, *t, "every tensor");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor ws = dispatch_ws(x.device(), nk, (int)el);
  check_rc(bgmoe_dispatch_scatter_ragged(ptr<uint16_t>(x), ptr<int32_t>(ids), (int)n, (int)k, (int)h, ptr<uint16_t>(act),
                                         act.size(0), (int)expert_start, (int)el, ptr<int32_t>(counts), ptr<int32_t>(counters),
                                         ptr<int32_t>(pos), ptr<int32_t>(cu), (int)row_align, ptr(ws),
                                         ws.defined() ? (size_t)ws.numel() : 0, cur_stream()));
  return {counts, cu, pos};
}

Tensor combine_fp32(Tensor y, Tensor pos, Tensor w, int64_t N, int64_t H, int64_t K, Tensor out) {
  TORCH_CHECK(N > 0 && H > 0, "N and H must be positive");
  TORCH_CHECK(K == 16, "K3 FP32 weighted combine requires K=16, got ", K);
  want(y, "expert_output", at::kBFloat16);
  want(pos, "topk_pos", at::kInt);
  want(w, "topk_weights", at::kFloat);
  want(out, "output", at::kFloat);
  TORCH_CHECK(pos.numel() >= N * K && w.numel() >= N * K, "topk_pos / topk_weights is smaller than N*K");
  TORCH_CHECK(out.dim() == 2 && out.size(0) >= N && out.size(1) == H, "output must have shape [N, H]");
  TORCH_CHECK(y.dim() == 2 && y.size(1) == H, "expert_output must have shape [rows, H]");
  for (auto* t : {&pos, &w, &out}) same_device(y, *t, "topk_pos / topk_weights / output");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  check_rc(bgmoe_reduce_weighted_scatter_fp32(ptr<uint16_t>(y), ptr<int32_t>(pos), ptr<float>(w), (int)N, (int)H, (int)K,
                                              ptr<float>(out), cur_stream()));
  return out;
}

Tensor combine_ordered(Tensor y, Tensor pos, Tensor ids, Tensor w, int64_t N, int64_t H, int64_t K, Tensor out) {
  TORCH_CHECK(N > 0 && H > 0, "N and H must be positive");
  TORCH_CHECK(K == 2 || K == 4 || K == 8, "ordered BF16 combine supports K=2,4,8, got ", K);
  TORCH_CHECK(H % 8 == 0, "ordered BF16 combine requires H % 8 == 0, got H=", H);
  want(y, "expert_output", at::kBFloat16);
  want(pos, "topk_pos", at::kInt);
  want(ids, "topk_indices", at::kInt);
  want(w, "topk_weights", at::kFloat);
  want(out, "output", at::kBFloat16);
  TORCH_CHECK(pos.numel() == N * K && ids.numel() == N * K && w.numel() == N * K, "topk_pos / topk_indices / topk_weights must "
              "contain N*K elements");
  TORCH_CHECK(out.numel() >= N * H, "output must have shape [N, H]");
  TORCH_CHECK(y.dim() == 2 && y.size(1) == H, "expert_output must have shape [rows, H]");
  for (auto* t : {&pos, &ids, &w, &out}) same_device(y, *t, "topk_pos / topk_indices / topk_weights / output");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  check_rc(bgmoe_reduce_weighted_scatter_bf16_ordered(ptr<uint16_t>(y), ptr<int32_t>(pos), ptr<int32_t>(ids), ptr<float>(w), (int)N,
                                                      (int)H, (int)K, ptr<uint16_t>(out), cur_stream()));
  return out;
}

// --------------------------------------------------------------------------------- _C_fp8_blockwise_gemm
struct Dims { int64_t m, n, k, m_pad, g; };
Dims check_gemm(const Tensor& x, const Tensor& weight, const Tensor& seqlens, const Tensor& cu, const Tensor& x_scale,
                const Tensor& w_scale, const char* wname) {
  want(x, "x");
  want(weight, wname);
  TORCH_CHECK(fp8_bytes(x) && fp8_bytes(weight), "x and ", wname, " must be float8_e4m3fn (or uint8 bytes)");
  want(seqlens, "seqlens", at::kInt);
  want(cu, "cu_seqlens", at::kInt);
  want(x_scale, "x_scale", at::kFloat);
  want(w_scale, "w_scale", at::kFloat);
  TORCH_CHECK(x.dim() == 2 && weight.dim() == 3 && x_scale.dim() == 2 && w_scale.dim() == 3, "x [m,K], weight [G,N,K], "
              "x_scale [K/128, m_pad], w_scale [G, N/128, pad4(K/128)] expected");
  Dims d{x.size(0), weight.size(1), x.size(1), x_scale.size(1), weight.size(0)};
  TORCH_CHECK(d.g > 0 && d.g <= 1024, "num_group must be in [1, 1024], got ", d.g);
  TORCH_CHECK(weight.size(2) == d.k, "x and weight K mismatch");
  TORCH_CHECK(d.k > 0 && d.k % 128 == 0 && d.n > 0 && d.n % 128 == 0, "K (", d.k, ") and N (", d.n, ") must be positive "
              "multiples of 128");
  TORCH_CHECK(seqlens.size(0) == d.g, "seqlens and weight num_group mismatch");
  TORCH_CHECK(cu.size(0) == d.g + 1, "cu_seqlens must have num_group + 1 entries, got ", cu.size(0));
  TORCH_CHECK(x_scale.size(0) == d.k / 128, "x_scale must have K/128 = ", d.k / 128, " rows, got ", x_scale.size(0));
  TORCH_CHECK(d.m > 0 && d.m_pad > 0 && d.m_pad <= d.m, "x_scale columns (m_pad=", d.m_pad, ") must be in [1, x rows=", d.m, "]");
  TORCH_CHECK(w_scale.size(0) == d.g && w_scale.size(1) == d.n / 128 && w_scale.size(2) >= d.k / 128,
              "w_scale must be [G, N/128, pad4(K/128)]");
  return d;
}
bgmoe_fp8_weight stacked(const Tensor& w, const Tensor& s) {
  bgmoe_fp8_weight d{};
  d.w = ptr<uint8_t>(w); d.w_group_stride = w.size(1) * w.size(2);
  d.scale = ptr<float>(s); d.scale_group_stride = s.size(1) * s.size(2); d.scale_nb_stride = s.size(2);
  d.layout = BGMOE_W_ROW_MAJOR;
  return d;
}
bgmoe_fp8_weight table(const Tensor& w_ptrs, const Tensor& s_proto, const Tensor& s_ptrs) {
  bgmoe_fp8_weight d{};
  d.w_ptrs = reinterpret_cast<const uint8_t* const*>(w_ptrs.data_ptr());
  d.scale_ptrs = reinterpret_cast<const float* const*>(s_ptrs.data_ptr());
  d.scale_nb_stride = s_proto.size(-1);
  d.layout = BGMOE_W_ROW_MAJOR;
  return d;
}
Tensor out_or_new(const OptTensor& output, const Tensor& x, int64_t m, int64_t n) {
  Tensor out = given(output) ? *output : torch::empty({m, n}, x.options().dtype(at::kBFloat16));
  want(out, "output", at::kBFloat16);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == m && out.size(1) == n, "output must be BF16 [m, N] = [", m, ", ", n, "]");
  return out;
}

Tensor grouped_gemm(Tensor x, Tensor weight, Tensor seqlens, Tensor cu, Tensor x_scale, Tensor w_scale, int64_t avg, OptTensor output,
                    OptTensor tma_desc, OptTensor tiles, OptTensor cu_tiles, bool update_tma) {
  (void)avg; (void)tma_desc; (void)tiles; (void)cu_tiles; (void)update_tma;     // row tiling is chosen on the device
  const Dims d = check_gemm(x, weight, seqlens, cu, x_scale, w_scale, "weight");
  Tensor out = out_or_new(output, x, d.m, d.n);
  bgmoe_fp8_act a{ptr<uint8_t>(x), ptr<float>(x_scale), 1, d.m_pad, 0};
  bgmoe_fp8_weight b = stacked(weight, w_scale);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_fp8_grouped_gemm(&a, &b, ptr<int32_t>(seqlens), ptr<int32_t>(cu), (int)d.g, d.m, (int)d.n, (int)d.k,
                                  ptr<uint16_t>(out), cur_stream()));
  return out;
}

Tensor fused_s1(Tensor x, Tensor gate, Tensor up, Tensor seqlens, Tensor cu, Tensor x_scale, Tensor gate_s, Tensor up_s, int64_t avg,
                OptTensor output, OptTensor tma_desc, OptTensor tiles, OptTensor cu_tiles, bool update_tma) {
  (void)avg; (void)tma_desc; (void)tiles; (void)cu_tiles; (void)update_tma;
  const Dims d = check_gemm(x, gate, seqlens, cu, x_scale, gate_s, "gate_weight");
  check_gemm(x, up, seqlens, cu, x_scale, up_s, "up_weight");
  TORCH_CHECK(gate.sizes() == up.sizes(), "gate_weight and up_weight shape mismatch");
  Tensor out = out_or_new(output, x, d.m, d.n);
  bgmoe_fp8_act a{ptr<uint8_t>(x), ptr<float>(x_scale), 1, d.m_pad, 0};
  bgmoe_fp8_weight wg = stacked(gate, gate_s), wu = stacked(up, up_s);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_fp8_fused_s1(&a, &wg, &wu, ptr<int32_t>(seqlens), ptr<int32_t>(cu), (int)d.g, d.m, (int)d.n, (int)d.k,
                              ptr<uint16_t>(out), nullptr, nullptr, 0, 0, cur_stream()));
  return out;
}

void check_ptrs(const Tensor& t, int64_t g, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kLong && t.dim() == 1 && t.numel() == g, name,
              " must be a CUDA int64 [", g, "] tensor of device pointers");
}
Tensor grouped_gemm_ptrs(Tensor x, Tensor w_proto, Tensor w_ptrs, Tensor seqlens, Tensor cu, Tensor x_scale, Tensor s_proto,
                         Tensor s_ptrs, int64_t avg, OptTensor output, OptTensor tma_desc, OptTensor tiles, OptTensor cu_tiles) {
  (void)avg; (void)tma_desc; (void)tiles; (void)cu_tiles;
  const int64_t g = seqlens.numel();
  check_ptrs(w_ptrs, g, "weight_ptrs");
  check_ptrs(s_ptrs, g, "w_scale_ptrs");
  const int64_t n = w_proto.size(-2), k = w_proto.size(-1), m = x.size(0);
  TORCH_CHECK(x.size(1) == k && k % 128 == 0 && n % 128 == 0, "x / weight_prototype K, N mismatch or not multiples of 128");
  want(x, "x");
  want(x_scale, "x_scale", at::kFloat);
  Tensor out = out_or_new(output, x, m, n);
  bgmoe_fp8_act a{ptr<uint8_t>(x), ptr<float>(x_scale), 1, x_scale.size(1), 0};
  bgmoe_fp8_weight b = table(w_ptrs, s_proto, s_ptrs);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_fp8_grouped_gemm(&a, &b, ptr<int32_t>(seqlens), ptr<int32_t>(cu), (int)g, m, (int)n, (int)k, ptr<uint16_t>(out),
                                  cur_stream()));
  return out;
}
Tensor fused_s1_ptrs(Tensor x, Tensor g_proto, Tensor g_ptrs, Tensor u_proto, Tensor u_ptrs, Tensor seqlens, Tensor cu, Tensor x_scale,
                     Tensor gs_proto, Tensor gs_ptrs, Tensor us_proto, Tensor us_ptrs, int64_t avg, OptTensor output,
                     OptTensor tma_desc, OptTensor tiles, OptTensor cu_tiles) {
  (void)avg; (void)tma_desc; (void)tiles; (void)cu_tiles; (void)u_proto;
  const int64_t g = seqlens.numel();
  for (auto* t : {&g_ptrs, &u_ptrs, &gs_ptrs, &us_ptrs}) check_ptrs(*t, g, "pointer table");
  const int64_t n = g_proto.size(-2), k = g_proto.size(-1), m = x.size(0);
  TORCH_CHECK(x.size(1) == k && k % 128 == 0 && n % 128 == 0, "x / gate_weight_prototype K, N mismatch or not multiples of 128");
  want(x, "x");
  want(x_scale, "x_scale", at::kFloat);
  Tensor out = out_or_new(output, x, m, n);
  bgmoe_fp8_act a{ptr<uint8_t>(x), ptr<float>(x_scale), 1, x_scale.size(1), 0};
  bgmoe_fp8_weight wg = table(g_ptrs, gs_proto, gs_ptrs), wu = table(u_ptrs, us_proto, us_ptrs);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_fp8_fused_s1(&a, &wg, &wu, ptr<int32_t>(seqlens), ptr<int32_t>(cu), (int)g, m, (int)n, (int)k, ptr<uint16_t>(out),
                              nullptr, nullptr, 0, 0, cur_stream()));
  return out;
}

// ---------------------------------------------------------------------------------- _C_fp8_blockwise_ops
std::vector<Tensor> act_quant_3d(Tensor x, Tensor tpe) {
  TORCH_CHECK(x.dim() == 3, "x must be 3D [E, mtp, K]");
  TORCH_CHECK(x.scalar_type() == at::kBFloat16, "x must be BF16");
  want(x, "x");
  want(tpe, "tokens_per_expert", at::kInt);
  const int64_t e = x.size(0), mtp = x.size(1), k = x.size(2);
  Tensor y = torch::empty({e, mtp, k}, x.options().dtype(at::kByte));
  Tensor s = torch::empty({e, mtp, (k + 127) / 128}, x.options().dtype(at::kFloat));
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_act_quant_3d(ptr<uint16_t>(x), ptr<int32_t>(tpe), (int)e, (int)mtp, (int)k, ptr<uint8_t>(y), ptr<float>(s),
                              cur_stream()));
  return {y, s};
}
std::vector<Tensor> act_quant_ragged(Tensor x, Tensor seqlens, Tensor cu, Tensor y, Tensor scale, int64_t row_align) {
  TORCH_CHECK(row_align > 0 && (row_align & (row_align - 1)) == 0, "row_align must be a positive power of two, got ", row_align);
  want(x, "x", at::kBFloat16);
  want(seqlens, "seqlens", at::kInt);
  want(cu, "cu_seqlens", at::kInt);
  want(y, "y");
  want(scale, "scale", at::kFloat);
  TORCH_CHECK(x.dim() == 2, "x must be BF16 [max_rows, K]");
  const int64_t rows = x.size(0), k = x.size(1), kb = (k + 127) / 128, e = seqlens.numel();
  TORCH_CHECK(seqlens.dim() == 1 && e >= 1, "seqlens must be int32 [E]");
  TORCH_CHECK(cu.dim() == 1 && cu.numel() == e + 1, "cu_seqlens must be int32 [E + 1]");
  TORCH_CHECK(fp8_bytes(y) && y.dim() == 2 && y.size(0) == rows && y.size(1) == k, "y must be uint8 or float8_e4m3fn [max_rows, K]");
  TORCH_CHECK(scale.dim() == 2 && scale.size(0) == kb && scale.size(1) == rows, "scale must be float32 [", kb, ", ", rows, "]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check_rc(bgmoe_act_quant_ragged(ptr<uint16_t>(x), ptr<int32_t>(seqlens), ptr<int32_t>(cu), (int)e, rows, (int)k, ptr<uint8_t>(y),
                                  ptr<float>(scale), (int)row_align, cur_stream()));
  return {y, scale};
}
Tensor silu_mul_3d(Tensor gate, Tensor up, Tensor tpe) {
  TORCH_CHECK(gate.dim() == 3 && up.dim() == 3, "Inputs must be 3D");
  TORCH_CHECK(gate.sizes() == up.sizes(), "Shape mismatch");
  want(gate, "gate", at::kBFloat16);
  want(up, "up", at::kBFloat16);
  want(tpe, "tokens_per_expert", at::kInt);
  Tensor out = torch::empty_like(gate);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(gate.device());
  check_rc(bgmoe_silu_mul_3d(ptr<uint16_t>(gate), ptr<uint16_t>(up), ptr<int32_t>(tpe), (int)gate.size(0), (int)gate.size(1),
                             (int)gate.size(2), ptr<uint16_t>(out), cur_stream()));
  return out;
}
std::vector<Tensor> fused_silu_quant_3d(Tensor gate, Tensor up, Tensor tpe) {
  TORCH_CHECK(gate.dim() == 3 && up.dim() == 3, "Inputs must be 3D");
  TORCH_CHECK(gate.sizes() == up.sizes(), "Shape mismatch");
  want(gate, "gate", at::kBFloat16);
  want(up, "up", at::kBFloat16);
  want(tpe, "tokens_per_expert", at::kInt);
  const int64_t e = gate.size(0), mtp = gate.size(1), n = gate.size(2);
  Tensor y = torch::empty({e, mtp, n}, gate.options().dtype(at::kByte));
  Tensor s = torch::empty({e, mtp, (n + 127) / 128}, gate.options().dtype(at::kFloat));
  c10::hip::HIPGuardMasqueradingAsCUDA guard(gate.device());
  check_rc(bgmoe_fused_silu_quant_3d(ptr<uint16_t>(gate), ptr<uint16_t>(up), ptr<int32_t>(tpe), (int)e, (int)mtp, (int)n,
                                     ptr<uint8_t>(y), ptr<float>(s), cur_stream()));
  return {y, s};
}
Tensor deepep_ll_scale_repack(Tensor recv, Tensor count, Tensor out, int64_t span_align) {
  TORCH_CHECK(recv.is_cuda() && recv.dim() == 3 && recv.scalar_type() == at::kFloat, "recv_scales must be float32 [E, S, hidden/128]");
  const int64_t e = recv.size(0), s = recv.size(1), kb = recv.size(2);
  TORCH_CHECK(e > 0 && s > 0 && kb > 0, "recv_scales must be non-empty");
  TORCH_CHECK(recv.stride(0) == kb * s && recv.stride(1) == 1 && recv.stride(2) == s, "recv_scales must be the (1, 2)-transposed view "
              "of a contiguous [E, hidden/128, S] block");
  want(count, "recv_count", at::kInt);
  TORCH_CHECK(count.dim() == 1 && count.size(0) == e, "recv_count must be int32 [E]");
  want(out, "out", at::kFloat);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == kb && out.size(1) == e * s, "out must be float32 [hidden/128, E * S]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(recv.device());
  static std::mutex mu;
  static std::map<int, Tensor> status;
  Tensor st;
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = status.find(recv.device().index());
    if (it == status.end()) it = status.emplace(recv.device().index(), torch::zeros({1}, count.options())).first;
    st = it->second;
  }
  check_rc(bgmoe_deepep_ll_scale_repack(ptr<float>(recv), ptr<int32_t>(count), ptr<float>(out), (int)e, (int)kb, (int)s, (int)span_align,
                                        ptr<int32_t>(st), cur_stream()));
  return out;
}

// --------------------------------------------------------------------------- _C_add_rmsnorm_fp8_quant
std::vector<Tensor> add_rmsnorm_fp8_quant_forward(Tensor residual, Tensor hidden, Tensor weight, double eps, OptTensor norm_nv,
                                                  OptTensor quant_nv, OptTensor row_mask, bool scale_tma_aligned) {
  for (auto* t : {&residual, &hidden, &weight}) {
    TORCH_CHECK(t->is_cuda(), "residual, hidden and weight must be CUDA");
    TORCH_CHECK(t->scalar_type() == at::kBFloat16, "fused add+RMSNorm+FP8 requires bf16 inputs, got ", t->scalar_type());
  }
  residual = residual.contiguous();
  hidden = hidden.contiguous();
  weight = weight.contiguous();
  const int64_t h = residual.size(-1);
  TORCH_CHECK(h % 128 == 0 && h >= 128 && h <= 8192, "fused add+RMSNorm+FP8 handles hidden sizes that are multiples of 128 up to "
              "8192; got hidden_size=", h);
  TORCH_CHECK(residual.numel() == hidden.numel(), "residual and hidden must have the same number of elements");
  TORCH_CHECK(weight.numel() == h, "weight must hold ", h, " elements, got ", weight.numel());
  const int64_t rows = residual.numel() / h, blocks = h / 128;
  Tensor normed = torch::empty_like(residual);
  Tensor quant = torch::empty({rows, h}, residual.options().dtype(at::kFloat8_e4m3fn));
  Tensor scale;
  if (scale_tma_aligned) {
    const int64_t aligned = (rows + 3) / 4 * 4;
    scale = torch::empty({blocks, aligned}, residual.options().dtype(at::kFloat)).transpose(0, 1).slice(0, 0, rows);
  } else {
    scale = torch::empty({rows, blocks}, residual.options().dtype(at::kFloat));
  }
  if (rows == 0) return {normed, residual, quant, scale};
  auto one = [](const OptTensor& t, const char* name) -> const int32_t* {
    if (!t.has_value() || !t->defined()) return nullptr;
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kInt && t->numel() == 1, name, " must be one CUDA int32");
    return reinterpret_cast<const int32_t*>(t->data_ptr());
  };
  const int32_t* nnv = one(norm_nv, "norm_num_valid_tokens");
  const int32_t* qnv = one(quant_nv, "quant_num_valid_tokens");
  TORCH_CHECK(nnv == nullptr || nnv == qnv, "norm_num_valid_tokens requires quant_num_valid_tokens to be the SAME tensor");
  Tensor mask;
  if (row_mask.has_value() && row_mask->defined()) {
    TORCH_CHECK(row_mask->is_cuda(), "row_valid_mask must be CUDA");
    TORCH_CHECK(row_mask->scalar_type() == residual.scalar_type(), "row_valid_mask dtype must match residual dtype");
    TORCH_CHECK(row_mask->numel() == rows, "row_valid_mask must have one entry per row");
    mask = row_mask->contiguous();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(residual.device());
  check_rc(bgmoe_add_rmsnorm_fp8_quant(ptr<uint16_t>(residual), ptr<uint16_t>(hidden), ptr<uint16_t>(weight), rows, (int)h, (float)eps,
                                       ptr<uint16_t>(normed), ptr<uint8_t>(quant), ptr<float>(scale), scale.stride(0), scale.stride(1),
                                       nnv, qnv, mask.defined() ? ptr<uint16_t>(mask) : nullptr, cur_stream()));
  return {normed, residual, quant, scale};
}

}  // namespace

PYBIND11_MODULE(_C_routing, m) {
  m.def("dispatch_count_gather", &dispatch_count_gather, "Dispatch: count + prefix sum + gather (gfx950)", py::arg("x"),
        py::arg("topk_indices"), py::arg("expert_start"), py::arg("num_local_experts"), py::arg("expert_counts"),
        py::arg("expert_offsets"), py::arg("expert_counters"), py::arg("dispatched_x"), py::arg("topk_pos"),
        py::arg("rank_token_counts") = c10::nullopt, py::arg("rows_per_rank") = c10::nullopt);
  m.def("gate_sigmoid_topk",
        [](Tensor logits, Tensor bias, int64_t k, double rsf, Tensor ids, Tensor w, OptTensor nv, OptTensor latent_out,
           c10::optional<int64_t> latent_offset, OptTensor rank_counts, c10::optional<int64_t> rows_per_rank) {
          return gate_impl(logits, bias, k, rsf, ids, w, nv, latent_out, latent_offset.value_or(0), rank_counts,
                           rows_per_rank.value_or(0), 1024, false);
        },
        "Gate: fused sigmoid + top-k + normalize + scale (gfx950)", py::arg("router_logits"), py::arg("e_score_correction"),
        py::arg("k"), py::arg("routed_scaling_factor"), py::arg("topk_indices"), py::arg("topk_weights"),
        py::arg("num_valid_tokens") = c10::nullopt, py::arg("latent_out") = c10::nullopt, py::arg("latent_offset") = c10::nullopt,
        py::arg("rank_token_counts") = c10::nullopt, py::arg("rows_per_rank") = c10::nullopt);
  m.def("gate_sigmoid_topk_warp",
        [](Tensor logits, Tensor bias, int64_t k, double rsf, Tensor ids, Tensor w, OptTensor nv, OptTensor rank_counts,
           c10::optional<int64_t> rows_per_rank) {
          return gate_impl(logits, bias, k, rsf, ids, w, nv, c10::nullopt, 0, rank_counts, rows_per_rank.value_or(0), 256, true);
        },
        "Gate, one wave per token (E <= 256), int32 or int64 ids (gfx950)", py::arg("router_logits"), py::arg("e_score_correction"),
        py::arg("k"), py::arg("routed_scaling_factor"), py::arg("topk_indices"), py::arg("topk_weights"),
        py::arg("num_valid_tokens") = c10::nullopt, py::arg("rank_token_counts") = c10::nullopt,
        py::arg("rows_per_rank") = c10::nullopt);
  m.def("glm5_router_gemm", &glm5_router_gemm, "GLM-5 router GEMM: BF16 hidden x BF16 weight^T -> FP32 logits (gfx950)",
        py::arg("hidden_states"), py::arg("router_weight"), py::arg("rank_token_counts"), py::arg("output"), py::arg("bucket_size"),
        py::arg("world_size"));
  m.def("reduce_weighted_scatter", &combine, "Reduce: weighted scatter-add (gfx950)", py::arg("expert_output"), py::arg("topk_pos"),
        py::arg("topk_weights"), py::arg("N"), py::arg("H"), py::arg("K"), py::arg("output"), py::arg("num_valid_tokens") = -1);
}

PYBIND11_MODULE(_C_mgn_ops, m) {
  m.def("moe_fused_gate", &moe_fused_gate, "Fused MoE gate: hierarchical group selection + top-k expert selection (gfx950)",
        py::arg("scores"), py::arg("e_score_correction_bias"), py::arg("n_group"), py::arg("topk_group"), py::arg("n_routed_experts"),
        py::arg("top_k"), py::arg("routed_scaling_factor"));
  m.def("expert_bincount", &expert_bincount, "Count tokens per expert + compact active expert metadata (gfx950)", py::arg("eids"),
        py::arg("routed_expert_start_idx"), py::arg("experts_per_rank"), py::arg("device"));
  m.def("fused_moe_token_dispatch", &fused_moe_token_dispatch, "Dispatch tokens to experts based on top-k indices (gfx950)",
        py::arg("global_x"), py::arg("topk_idx"), py::arg("token_idx"), py::arg("topk_pos"), py::arg("routed_expert_start_idx"),
        py::arg("routed_expert_end_idx"));
  m.def("compact_expert_data", &compact_expert_data, "Compact expert counts into dense active-expert metadata (gfx950)",
        py::arg("expert_counts"));
}

PYBIND11_MODULE(_C_dispatch_scatter_3d, m) {
  m.def("dispatch_scatter_3d", &dispatch_scatter_3d, "3D dispatch scatter for strided MoE buffer layout");
  m.def("dispatch_scatter_ragged", &dispatch_scatter_ragged, "Compact ragged dispatch scatter with aligned device cu_seqlens");
  m.def("reduce_weighted_scatter",
        [](Tensor y, Tensor pos, Tensor w, int64_t N, int64_t H, int64_t K, Tensor out) { return combine(y, pos, w, N, H, K, out, -1); },
        "Weighted reduce scatter from 3D to flat layout");
  m.def("reduce_weighted_scatter_fp32", &combine_fp32, "K=16 weighted reduction with FP32 output");
  m.def("reduce_weighted_scatter_bf16_ordered", &combine_ordered, "Expert-id-ordered weighted reduction with BF16 rounding per step");
}

PYBIND11_MODULE(_C_fp8_blockwise_gemm, m) {
  m.def("fp8_blockwise_grouped_gemm", &grouped_gemm, "FP8 blockwise grouped GEMM (gfx950 MFMA)", py::arg("x"), py::arg("weight"),
        py::arg("seqlens"), py::arg("cu_seqlens"), py::arg("x_scale"), py::arg("w_scale"), py::arg("num_seq_per_group_avg"),
        py::arg("output") = py::none(), py::arg("tma_desc") = py::none(), py::arg("tiles") = py::none(),
        py::arg("cu_tiles") = py::none(), py::arg("update_tma") = true);
  m.def("fp8_blockwise_grouped_gemm_ptrs", &grouped_gemm_ptrs, "FP8 blockwise grouped GEMM over independent weight pointer arrays",
        py::arg("x"), py::arg("weight_prototype"), py::arg("weight_ptrs"), py::arg("seqlens"), py::arg("cu_seqlens"),
        py::arg("x_scale"), py::arg("w_scale_prototype"), py::arg("w_scale_ptrs"), py::arg("num_seq_per_group_avg"),
        py::arg("output") = py::none(), py::arg("tma_desc") = py::none(), py::arg("tiles") = py::none(),
        py::arg("cu_tiles") = py::none());
  m.def("fp8_blockwise_fused_s1", &fused_s1, "FP8 blockwise fused S1: gate + up + SiLU (gfx950 MFMA)", py::arg("x"),
        py::arg("gate_weight"), py::arg("up_weight"), py::arg("seqlens"), py::arg("cu_seqlens"), py::arg("x_scale"),
        py::arg("gate_w_scale"), py::arg("up_w_scale"), py::arg("num_seq_per_group_avg"), py::arg("output") = py::none(),
        py::arg("tma_desc") = py::none(), py::arg("tiles") = py::none(), py::arg("cu_tiles") = py::none(),
        py::arg("update_tma") = true);
  m.def("fp8_blockwise_prepare_s1_s3_tma",
        [](Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, int64_t, Tensor, Tensor, Tensor, Tensor) {},
        "No descriptors to prepare on gfx950 (row tiling is chosen on the device): accepted and ignored", py::arg("s1_x"),
        py::arg("s1_output"), py::arg("s3_x"), py::arg("s3_output"), py::arg("seqlens"), py::arg("cu_seqlens"),
        py::arg("num_seq_per_group_avg"), py::arg("s1_tma_desc"), py::arg("s3_tma_desc"), py::arg("tiles"), py::arg("cu_tiles"));
  m.def("fp8_blockwise_fused_s1_ptrs", &fused_s1_ptrs, "FP8 fused S1 over independent gate/up weight pointer arrays", py::arg("x"),
        py::arg("gate_weight_prototype"), py::arg("gate_weight_ptrs"), py::arg("up_weight_prototype"), py::arg("up_weight_ptrs"),
        py::arg("seqlens"), py::arg("cu_seqlens"), py::arg("x_scale"), py::arg("gate_w_scale_prototype"), py::arg("gate_w_scale_ptrs"),
        py::arg("up_w_scale_prototype"), py::arg("up_w_scale_ptrs"), py::arg("num_seq_per_group_avg"), py::arg("output") = py::none(),
        py::arg("tma_desc") = py::none(), py::arg("tiles") = py::none(), py::arg("cu_tiles") = py::none());
}

PYBIND11_MODULE(_C_fp8_blockwise_ops, m) {
  m.def("act_quant_3d", &act_quant_3d, "Per-token-group FP8 quantisation on the masked layout");
  m.def("act_quant_ragged", &act_quant_ragged, "Per-token-group FP8 quantisation on the ragged layout");
  m.def("silu_mul_3d", &silu_mul_3d, "silu(gate) * up on the masked layout");
  m.def("fused_silu_quant_3d", &fused_silu_quant_3d, "silu(gate) * up + FP8 quantisation on the masked layout");
  m.def("deepep_ll_scale_repack", &deepep_ll_scale_repack, "Span-limited repack of the low-latency exchange's scale block");
}

PYBIND11_MODULE(_C_add_rmsnorm_fp8_quant, m) {
  m.def("add_rmsnorm_fp8_quant_forward", &add_rmsnorm_fp8_quant_forward, "Fused add + RMSNorm + per-token 128-block e4m3fn cast",
        py::arg("residual"), py::arg("hidden"), py::arg("weight"), py::arg("eps"), py::arg("norm_num_valid_tokens") = c10::nullopt,
        py::arg("quant_num_valid_tokens") = c10::nullopt, py::arg("row_valid_mask") = c10::nullopt,
        py::arg("scale_tma_aligned") = false);
}
