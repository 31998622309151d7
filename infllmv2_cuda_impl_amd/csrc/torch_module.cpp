// The native module of the package, `infllmv2_cuda_impl_amd._C` (exposed as `infllm_v2.C`): a thin PyTorch C++
// extension over the C ABI of libinfllmv2_hip.so.  It binds the names, argument order and results of the
// reference's pybind module (csrc/entry.cu:197-215):
//
//   * the raw-pointer group (entry.cu:31-195): `topk`, `blockmask_to_uint64`, `topk_to_uint64`, `uint64_to_bool`,
//     `max_pooling_1d`, `max_pooling_1d_varlen` take uintptr_t pointers and a stream handle, return nothing and
//     are asynchronous on the given stream;
//   * the tensor group (entry.cu:13-18, 209-214): `fwd`, `varlen_fwd`, `varlen_fwd_stage1`, `bwd`, `varlen_bwd`,
//     `fwd_kvcache` take at::Tensor arguments in the layouts the reference's Python wrappers produce - on the
//     sparse path q / out / dout re-laid-out as (total_q * 16, Hk, d) with cu_seqlens_q and max_seqlen_q
//     multiplied by 16 - and are served by the same kernels through strides, without a copy.
//
// Host code only: no kernels live here.  Tensors are used for device memory, shapes and the current stream;
// every computation is one call into the C ABI declared in infllmv2_hip.h.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <optional>
#include <string>
#include <vector>

#include "infllmv2_hip.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;
constexpr int kGroup = 16;

void check_rc(int rc, const char* what) {
    if (rc != 0) {
        const char* msg = infllmv2_last_error();
        TORCH_CHECK(false, (msg && msg[0]) ? std::string(msg) : std::string(what) + " failed");
    }
}

// PyTorch on ROCm presents its HIP devices under the device type "cuda": guard and stream are the ones that go with it
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.get_device()).stream(); }

const void* cptr(const OptTensor& t) { return t.has_value() ? t->data_ptr() : nullptr; }

bool is_half(const Tensor& t) { return t.scalar_type() == at::kHalf; }

void require_gpu(const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must be on a GPU device; this library has no CPU path");
    check_rc(infllmv2_check_device(t.get_device()), "infllmv2_check_device");
}

// ---- raw-pointer group (entry.cu:31-195) ---------------------------------------------------------------------------
void topk(uintptr_t stream, int num_tokens, int dim, int top, int dtype, uintptr_t x, uintptr_t topk_val, uintptr_t topk_pos) {
    check_rc(infllmv2_topk(reinterpret_cast<void*>(stream), num_tokens, dim, top, dtype, reinterpret_cast<const void*>(x),
                           reinterpret_cast<void*>(topk_val), reinterpret_cast<int32_t*>(topk_pos)), "topk");
}
void blockmask_to_uint64(uintptr_t stream, uintptr_t blockmask, uintptr_t result, int64_t batch_size, int last_dim_size,
                         int n_uint64_per_row) {
    check_rc(infllmv2_blockmask_to_uint64(reinterpret_cast<void*>(stream), reinterpret_cast<const uint8_t*>(blockmask),
                                          reinterpret_cast<uint64_t*>(result), batch_size, last_dim_size, n_uint64_per_row),
             "blockmask_to_uint64");
}
void topk_to_uint64(uintptr_t stream, uintptr_t topk_idx, uintptr_t result, int64_t batch_size, int k, int k_blocks,
                    int n_uint64_per_row) {
    check_rc(infllmv2_topk_to_uint64(reinterpret_cast<void*>(stream), reinterpret_cast<const int32_t*>(topk_idx),
                                     reinterpret_cast<uint64_t*>(result), batch_size, k, k_blocks, n_uint64_per_row),
             "topk_to_uint64");
}
void uint64_to_bool(uintptr_t stream, uintptr_t input, uintptr_t result, int64_t batch_size, int last_dim_size,
                    int n_uint64_per_row) {
    check_rc(infllmv2_uint64_to_bool(reinterpret_cast<void*>(stream), reinterpret_cast<const uint64_t*>(input),
                                     reinterpret_cast<uint8_t*>(result), batch_size, last_dim_size, n_uint64_per_row),
             "uint64_to_bool");
}
void max_pooling_1d(uintptr_t stream, uintptr_t input, uintptr_t output, int dtype, int num_heads, int q_len, int k_len,
                    int out_len, int cache_len, int kernel_size, int stride, int padding, int block_size, int local_blocks,
                    int init_blocks) {
    check_rc(infllmv2_max_pooling_1d(reinterpret_cast<void*>(stream), reinterpret_cast<const void*>(input),
                                     reinterpret_cast<void*>(output), dtype, num_heads, q_len, k_len, out_len, cache_len,
                                     kernel_size, stride, padding, block_size, local_blocks, init_blocks), "max_pooling_1d");
}
void max_pooling_1d_varlen(uintptr_t stream, uintptr_t input, uintptr_t output, uintptr_t cu_seqlens_q, uintptr_t cu_seqlens_k,
                           uintptr_t cache_lens, int dtype, int batch_size, int num_heads, int max_seqlen_q, int max_seqlen_k,
                           int out_len, int kernel_size, int stride, int padding, int block_size, int local_blocks,
                           int init_blocks) {
    check_rc(infllmv2_max_pooling_1d_varlen(reinterpret_cast<void*>(stream), reinterpret_cast<const void*>(input),
                                            reinterpret_cast<void*>(output), reinterpret_cast<const int32_t*>(cu_seqlens_q),
                                            reinterpret_cast<const int32_t*>(cu_seqlens_k),
                                            reinterpret_cast<const int32_t*>(cache_lens), dtype, batch_size, num_heads,
                                            max_seqlen_q, max_seqlen_k, out_len, kernel_size, stride, padding, block_size,
                                            local_blocks, init_blocks), "max_pooling_1d_varlen");
}
void get_probs(py::args, py::kwargs) {
    PyErr_SetString(PyExc_NotImplementedError, "get_probs is bound by the reference but unused by its package; not built here");
    throw py::error_already_set();
}

// ---- helpers of the tensor group -------------------------------------------------------------------------------------
// Options the reference build compiles out fail with its messages (flash_api.cpp:107-109, 131-133, 144-147, 330-332).
// Returns the causal flag of the launch, derived from the window the way the reference derives it (flash_api.cpp:137,
// 600, 621-622).
bool launch_causal(double p_dropout, int64_t wl, int64_t wr, double softcap, const OptTensor& alibi, bool causal,
                   int64_t max_seqlen_k) {
    TORCH_CHECK(!(softcap > 0.0), "This flash attention build does not support softcap.");
    TORCH_CHECK(p_dropout < 1.0, "Expected p_dropout < 1.f to be true, but got false.");
    TORCH_CHECK(p_dropout == 0.0, "This flash attention build does not support dropout.");
    if (max_seqlen_k >= 0) {
        if (wl >= max_seqlen_k) wl = -1;
        if (wr >= max_seqlen_k) wr = -1;
    }
    if (causal) wr = 0;
    const bool is_causal = wl < 0 && wr == 0;
    TORCH_CHECK(is_causal || (wl < 0 && wr < 0), "This flash attention build does not support local attention.");
    TORCH_CHECK(!alibi.has_value(), "This flash attention build does not support alibi.");
    return is_causal;
}

void common_checks(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& cu_q, const Tensor& cu_k) {
    TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16,
                "FlashAttention only support fp16 and bf16 data type");
    TORCH_CHECK(k.scalar_type() == q.scalar_type(), "query and key must have the same dtype");
    TORCH_CHECK(v.scalar_type() == q.scalar_type(), "query and value must have the same dtype");
    TORCH_CHECK(cu_q.scalar_type() == at::kInt, "cu_seqlens_q must have dtype int32");
    TORCH_CHECK(cu_k.scalar_type() == at::kInt, "cu_seqlens_k must have dtype int32");
    require_gpu(q, "q"); require_gpu(k, "k"); require_gpu(v, "v"); require_gpu(cu_q, "cu_seqlens_q"); require_gpu(cu_k, "cu_seqlens_k");
    TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, "q, k, v must have shape (total, num_heads, head_size)");
    TORCH_CHECK(cu_q.is_contiguous() && cu_k.is_contiguous(), "cu_seqlens must be contiguous");
    TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1, "Input tensor must have contiguous last dimension");
    TORCH_CHECK(cu_q.numel() - 1 > 0, "batch size must be positive");
}

struct Strides3 { int64_t v[3]; };
struct Strides2 { int64_t v[2]; };
// {token, head-in-group, kv-head} strides of a q-like tensor: (T*16, Hk, d) when expanded, else (T, Hq, d)
Strides3 q_layout(const Tensor& t, bool expanded) {
    if (expanded) return {{kGroup * t.stride(0), t.stride(0), t.stride(1)}};
    return {{t.stride(0), t.stride(1), kGroup * t.stride(1)}};
}
Strides2 kv_layout(const Tensor& t) { return {{t.stride(0), t.stride(1)}}; }

Tensor bytes_on(const Tensor& like, size_t n) {
    return at::empty({static_cast<int64_t>(n < 256 ? 256 : n)}, like.options().dtype(at::kByte));
}

// ---- tensor group ----------------------------------------------------------------------------------------------------
// mha_varlen_fwd (flash_api.cpp:519-782).  Returns {out, softmax_lse, p, rng_state}.
std::vector<Tensor> varlen_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& out_, const Tensor& cu_seqlens_q,
                               const Tensor& cu_seqlens_k, const OptTensor& seqused_k, const OptTensor& leftpad_k_,
                               const OptTensor& block_table_, const OptTensor& alibi_slopes_, int64_t max_seqlen_q,
                               int64_t max_seqlen_k, double p_dropout, double softmax_scale, bool zero_tensors, bool is_causal,
                               int64_t window_size_left, int64_t window_size_right, double softcap, bool return_softmax,
                               const py::object& gen_, const OptTensor& blockmask_) {
    (void)zero_tensors; (void)gen_;
    common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k);
    is_causal = launch_causal(p_dropout, window_size_left, window_size_right, softcap, alibi_slopes_, is_causal, max_seqlen_k);
    TORCH_CHECK(!seqused_k.has_value(), "seqused_k is not supported by this build");
    TORCH_CHECK(!leftpad_k_.has_value(), "leftpad_k is not supported by this build");
    TORCH_CHECK(!block_table_.has_value(), "block_table is not supported by this build");
    TORCH_CHECK(!return_softmax, "return_softmax is only supported when p_dropout > 0.0");
    DeviceGuard guard(q.device());
    const int64_t Hk = k.size(1);
    const bool expanded = blockmask_.has_value() && q.size(1) == Hk;
    const int batch = static_cast<int>(cu_seqlens_q.numel() - 1);
    int64_t total_q, Hq, max_q;
    Tensor cu_q, lse;
    int64_t lse_strides[3];
    if (expanded) {
        TORCH_CHECK(q.size(0) % kGroup == 0 && max_seqlen_q % kGroup == 0, "the re-laid-out query must hold 16 rows per token");
        total_q = q.size(0) / kGroup; Hq = Hk * kGroup; max_q = max_seqlen_q / kGroup;
        cu_q = at::div(cu_seqlens_q, kGroup, "floor").to(at::kInt);
        lse = at::empty({Hk, total_q * kGroup}, q.options().dtype(at::kFloat));
        lse_strides[0] = kGroup; lse_strides[1] = 1; lse_strides[2] = total_q * kGroup;
    } else {
        total_q = q.size(0); Hq = q.size(1); max_q = max_seqlen_q;
        cu_q = cu_seqlens_q;
        lse = at::empty({Hq, total_q}, q.options().dtype(at::kFloat));
        lse_strides[0] = 1; lse_strides[1] = total_q; lse_strides[2] = kGroup * total_q;
    }
    if (max_q == 1) is_causal = false;                                  // flash_api.cpp:599
    Tensor out = out_.has_value() ? *out_ : at::empty_like(q);
    TORCH_CHECK(out.scalar_type() == q.scalar_type(), "Output must have the same dtype as inputs");
    TORCH_CHECK(out.sizes() == q.sizes(), "out must have the shape of q");
    const int64_t total_k = k.size(0);
    Tensor ws = bytes_on(q, infllmv2_kv_image_bytes(total_k, batch, static_cast<int>(Hk)));
    const int n64 = blockmask_.has_value() ? static_cast<int>(blockmask_->size(-1)) : 0;
    const Strides3 qs = q_layout(q, expanded), os = q_layout(out, expanded);
    const Strides2 ks = kv_layout(k), vs = kv_layout(v);
    auto fn = is_half(q) ? infllmv2_varlen_fwd_f16 : infllmv2_varlen_fwd;
    check_rc(fn(stream_of(q), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr<float>(),
                cu_q.data_ptr<int32_t>(), cu_seqlens_k.data_ptr<int32_t>(), static_cast<const uint64_t*>(cptr(blockmask_)),
                ws.data_ptr(), static_cast<size_t>(ws.numel()), 0, batch, total_q, total_k, static_cast<int>(Hq),
                static_cast<int>(Hk), static_cast<int>(q.size(-1)), static_cast<int>(max_q), static_cast<int>(max_seqlen_k),
                qs.v, ks.v, vs.v, os.v, lse_strides, n64, static_cast<float>(softmax_scale), is_causal ? 1 : 0), "varlen_fwd");
    Tensor p = at::empty({0}, q.options());
    Tensor rng_state = at::empty({2}, q.options().dtype(at::kLong));
    return {out, lse, p, rng_state};
}

// mha_varlen_fwd_stage1 (flash_api.cpp:784-1049): q is the re-laid-out (T*16, Hk, d) tensor.  Returns {p} with p
// (Hk, T, round128(max_seqlen_k)) like the reference's buffer (flash_api.cpp:941); columns >= max_seqlen_k are zero.
std::vector<Tensor> varlen_fwd_stage1(const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& out_,
                                      const Tensor& cu_seqlens_q, const Tensor& cu_seqlens_k, const Tensor& cu_seqlens_v,
                                      const OptTensor& seqused_k, const OptTensor& leftpad_k_, const OptTensor& block_table_,
                                      const OptTensor& alibi_slopes_, int64_t max_seqlen_q, int64_t max_seqlen_k,
                                      double p_dropout, double softmax_scale, bool zero_tensors, bool is_causal,
                                      int64_t window_size_left, int64_t window_size_right, double softcap,
                                      bool return_softmax, const py::object& gen_) {
    (void)out_; (void)seqused_k; (void)leftpad_k_; (void)block_table_; (void)zero_tensors; (void)return_softmax; (void)gen_;
    common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k);
    is_causal = launch_causal(p_dropout, window_size_left, window_size_right, softcap, alibi_slopes_, is_causal, max_seqlen_k);
    DeviceGuard guard(q.device());
    const int64_t Hk = k.size(1);
    TORCH_CHECK(q.size(1) == Hk && q.size(0) % kGroup == 0,
                "stage 1 expects the query re-laid-out as (total_q * 16, num_heads_k, head_size)");
    const int64_t total_q = q.size(0) / kGroup;
    const int batch = static_cast<int>(cu_seqlens_q.numel() - 1);
    Tensor cu_q = at::div(cu_seqlens_q, kGroup, "floor").to(at::kInt);
    const int64_t row = (max_seqlen_k + 127) / 128 * 128;
    Tensor p = row != max_seqlen_k ? at::zeros({Hk, total_q, row}, q.options()) : at::empty({Hk, total_q, row}, q.options());
    const Strides3 qs = q_layout(q, true);
    const Strides2 ks = kv_layout(k), vs = kv_layout(v);
    auto fn = is_half(q) ? infllmv2_varlen_fwd_stage1_f16 : infllmv2_varlen_fwd_stage1;
    check_rc(fn(stream_of(q), q.data_ptr(), k.data_ptr(), v.data_ptr(), p.data_ptr(), cu_q.data_ptr<int32_t>(),
                cu_seqlens_k.data_ptr<int32_t>(), cu_seqlens_v.data_ptr<int32_t>(), batch, total_q, static_cast<int>(Hk * kGroup),
                static_cast<int>(Hk), static_cast<int>(q.size(-1)), static_cast<int>(max_seqlen_q / kGroup),
                static_cast<int>(max_seqlen_k), qs.v, ks.v, vs.v, p.stride(0), p.stride(1), static_cast<float>(softmax_scale),
                is_causal ? 1 : 0), "varlen_fwd_stage1");
    return {p};
}

// mha_varlen_bwd (flash_api.cpp:1278-1547).  col_blockmask_ is the transposed mask (Hk, k_blocks, ceil(T/64)) the
// reference's Python wrapper builds; it is turned back into the row mask (the dQ kernel walks rows, the dK/dV kernel
// re-derives the columns).  dq, dk, dv are written in place and returned with an empty softmax_d.
std::vector<Tensor> varlen_bwd(const Tensor& dout, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& out,
                               const Tensor& softmax_lse, const OptTensor& dq_, const OptTensor& dk_, const OptTensor& dv_,
                               const Tensor& cu_seqlens_q, const Tensor& cu_seqlens_k, const OptTensor& alibi_slopes_,
                               int64_t max_seqlen_q, int64_t max_seqlen_k, double p_dropout, double softmax_scale,
                               bool zero_tensors, bool is_causal, int64_t window_size_left, int64_t window_size_right,
                               double softcap, bool deterministic, const OptTensor& col_blockmask_, const py::object& gen_,
                               const OptTensor& rng_state) {
    (void)zero_tensors; (void)gen_; (void)rng_state;
    common_checks(q, k, v, cu_seqlens_q, cu_seqlens_k);
    is_causal = launch_causal(p_dropout, window_size_left, window_size_right, softcap, alibi_slopes_, is_causal, max_seqlen_k);
    DeviceGuard guard(q.device());
    const int64_t Hk = k.size(1);
    const bool expanded = col_blockmask_.has_value() && q.size(1) == Hk;
    const int batch = static_cast<int>(cu_seqlens_q.numel() - 1);
    int64_t total_q, Hq, max_q;
    Tensor cu_q;
    int64_t lse_strides[3];
    if (expanded) {
        total_q = q.size(0) / kGroup; Hq = Hk * kGroup; max_q = max_seqlen_q / kGroup;
        cu_q = at::div(cu_seqlens_q, kGroup, "floor").to(at::kInt);
        lse_strides[0] = kGroup; lse_strides[1] = 1; lse_strides[2] = total_q * kGroup;
    } else {
        total_q = q.size(0); Hq = q.size(1); max_q = max_seqlen_q;
        cu_q = cu_seqlens_q;
        lse_strides[0] = 1; lse_strides[1] = total_q; lse_strides[2] = kGroup * total_q;
    }
    Tensor dq = dq_.has_value() ? *dq_ : at::empty_like(q);
    Tensor dk = dk_.has_value() ? *dk_ : at::empty_like(k);
    Tensor dv = dv_.has_value() ? *dv_ : at::empty_like(v);
    Tensor fwd_mask;
    int n64 = 0;
    if (col_blockmask_.has_value()) {
        const int64_t k_blocks = (max_seqlen_k + 63) / 64;
        TORCH_CHECK(col_blockmask_->dim() == 3 && col_blockmask_->scalar_type() == at::kLong,
                    "col_blockmask must be an int64 tensor of shape (num_heads_k, k_blocks, ceil(total_q / 64))");
        TORCH_CHECK(col_blockmask_->size(1) >= k_blocks, "col_blockmask has fewer rows than key blocks");
        Tensor cols = col_blockmask_->slice(1, 0, k_blocks).contiguous();           // rows <-> columns
        const int64_t n64_out = (k_blocks + 63) / 64;
        fwd_mask = at::empty({cols.size(0), total_q, n64_out}, cols.options());
        check_rc(infllmv2_transpose_blockmask(stream_of(q), reinterpret_cast<const uint64_t*>(cols.data_ptr()),
                                              reinterpret_cast<uint64_t*>(fwd_mask.data_ptr()), static_cast<int>(cols.size(0)),
                                              cols.size(1), static_cast<int>(cols.size(2)), static_cast<int>(total_q),
                                              static_cast<int>(n64_out)), "transpose_blockmask");
        n64 = static_cast<int>(n64_out);
    }
    const int64_t total_k = k.size(0);
    const size_t ws_bytes = deterministic
        ? infllmv2_varlen_bwd_deterministic_workspace_bytes(batch, total_q, total_k, static_cast<int>(Hk), static_cast<int>(max_seqlen_k))
        : infllmv2_varlen_bwd_workspace_bytes(batch, total_q, total_k, static_cast<int>(Hk), static_cast<int>(max_seqlen_k));
    Tensor ws = bytes_on(q, ws_bytes);
    const Strides3 qs = q_layout(q, expanded), os = q_layout(out, expanded), dos = q_layout(dout, expanded), dqs = q_layout(dq, expanded);
    const Strides2 ks = kv_layout(k), vs = kv_layout(v), dks = kv_layout(dk), dvs = kv_layout(dv);
    auto fn = is_half(q) ? infllmv2_varlen_bwd_f16 : infllmv2_varlen_bwd;
    check_rc(fn(stream_of(q), dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                softmax_lse.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cu_q.data_ptr<int32_t>(),
                cu_seqlens_k.data_ptr<int32_t>(), fwd_mask.defined() ? reinterpret_cast<const uint64_t*>(fwd_mask.data_ptr()) : nullptr,
                ws.data_ptr(), static_cast<size_t>(ws.numel()), batch, total_q, total_k, static_cast<int>(Hq), static_cast<int>(Hk),
                static_cast<int>(q.size(-1)), static_cast<int>(max_q), static_cast<int>(max_seqlen_k), qs.v, ks.v, vs.v, os.v,
                dos.v, dqs.v, dks.v, dvs.v, lse_strides, n64, static_cast<float>(softmax_scale), is_causal ? 1 : 0,
                deterministic ? 1 : 0), "varlen_bwd");
    return {dq, dk, dv, at::empty({0}, q.options().dtype(at::kFloat))};
}

// mha_fwd_kvcache (flash_api.cpp:1549-1843).  Returns {out, softmax_lse}.  The option conflicts and alignment rules
// are checked by the C entry point with the reference's messages; what needs tensor shapes is checked here.
std::vector<Tensor> fwd_kvcache(const Tensor& q, const Tensor& kcache, const Tensor& vcache, const OptTensor& k_,
                                const OptTensor& v_, const OptTensor& seqlens_k_, const OptTensor& rotary_cos_,
                                const OptTensor& rotary_sin_, const OptTensor& cache_batch_idx_, const OptTensor& leftpad_k_,
                                const OptTensor& block_table_, const OptTensor& alibi_slopes_, const OptTensor& out_,
                                double softmax_scale, bool is_causal, int64_t window_size_left, int64_t window_size_right,
                                double softcap, bool is_rotary_interleaved, int64_t num_splits, const OptTensor& blockmask_) {
    launch_causal(0.0, window_size_left, window_size_right, softcap, alibi_slopes_, is_causal, -1);
    require_gpu(q, "q"); require_gpu(kcache, "k_cache"); require_gpu(vcache, "v_cache");
    TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "FlashAttention only support fp16 and bf16 data type");
    TORCH_CHECK(kcache.scalar_type() == q.scalar_type(), "query and key must have the same dtype");
    TORCH_CHECK(vcache.scalar_type() == q.scalar_type(), "query and value must have the same dtype");
    TORCH_CHECK(q.dim() == 4 && kcache.dim() == 4 && vcache.dim() == 4, "q, k_cache, v_cache must have 4 dimensions");
    TORCH_CHECK(q.stride(-1) == 1 && kcache.stride(-1) == 1 && vcache.stride(-1) == 1, "Input tensor must have contiguous last dimension");
    DeviceGuard guard(q.device());
    const int batch = static_cast<int>(q.size(0)), seqlen_q = static_cast<int>(q.size(1));
    const int Hq = static_cast<int>(q.size(2)), d = static_cast<int>(q.size(3)), Hk = static_cast<int>(kcache.size(2));
    const bool paged = block_table_.has_value();
    int cap, page = 0;
    int64_t table_stride = 0;
    if (paged) {
        TORCH_CHECK(block_table_->scalar_type() == at::kInt, "block_table must have dtype torch.int32");
        TORCH_CHECK(block_table_->stride(-1) == 1, "block_table must have contiguous last dimension");
        TORCH_CHECK(block_table_->dim() == 2 && block_table_->size(0) == batch,
                    "block_table must have shape (batch_size, max_num_blocks_per_seq)");
        page = static_cast<int>(kcache.size(1));
        cap = static_cast<int>(block_table_->size(1)) * page;
        table_stride = block_table_->stride(0);
        TORCH_CHECK(vcache.sizes() == kcache.sizes(),
                    "paged k_cache and v_cache must have shape (num_blocks, page_block_size, num_heads_k, head_size)");
    } else {
        cap = static_cast<int>(kcache.size(1));
        TORCH_CHECK(vcache.sizes() == kcache.sizes() && kcache.size(3) == d &&
                    (cache_batch_idx_.has_value() || kcache.size(0) == batch),
                    "k_cache and v_cache must have shape (batch_size, seqlen_cache, num_heads_k, head_size)");
    }
    int seqlen_new = 0;
    if (k_.has_value()) {
        TORCH_CHECK(v_.has_value(), "If key is supplied, value must also be passed in");
        TORCH_CHECK(k_->scalar_type() == q.scalar_type() && v_->scalar_type() == q.scalar_type(),
                    "Key and value must have the same dtype as query");
        seqlen_new = static_cast<int>(k_->size(1));
        TORCH_CHECK(k_->dim() == 4 && k_->size(0) == batch && k_->size(2) == Hk && k_->size(3) == d && v_->sizes() == k_->sizes(),
                    "k and v must have shape (batch_size, seqlen_new, num_heads_k, head_size)");
        TORCH_CHECK(seqlens_k_.has_value(), "If key is supplied, seqlens_k must also be passed in");
    }
    auto int_vec = [&](const OptTensor& t, const char* name) -> Tensor {
        if (!t.has_value()) return Tensor();
        TORCH_CHECK(t->scalar_type() == at::kInt, name, " must have dtype int32");
        TORCH_CHECK(t->dim() == 1 && t->size(0) == batch, name, " must have shape (batch_size)");
        return t->contiguous();
    };
    Tensor seqlens = int_vec(seqlens_k_, "seqlens_k"), batch_idx = int_vec(cache_batch_idx_, "cache_batch_idx"),
           leftpad = int_vec(leftpad_k_, "leftpad_k");
    int rotary_dim = 0;
    if (rotary_cos_.has_value()) {
        TORCH_CHECK(k_.has_value(), "If rotary cos/sin are provided, new key / value to be appended to KV cache must also be provided");
        TORCH_CHECK(rotary_sin_.has_value(), "If rotary cos is provided, rotary sin must also be provided");
        rotary_dim = static_cast<int>(rotary_cos_->size(1)) * 2;
        TORCH_CHECK(rotary_dim <= d, "rotary_dim must be <= headdim");
        TORCH_CHECK(rotary_dim % 16 == 0, "Only rotary dimensions divisible by 16 are currently supported");
        TORCH_CHECK(rotary_cos_->size(0) >= cap, "cos/sin seqlen must be at least the seqlen of KV cache");
        TORCH_CHECK(rotary_sin_->sizes() == rotary_cos_->sizes() && rotary_cos_->is_contiguous() && rotary_sin_->is_contiguous(),
                    "rotary_cos and rotary_sin must be contiguous (seqlen_ro, rotary_dim / 2) tensors");
        TORCH_CHECK(rotary_cos_->scalar_type() == q.scalar_type() && rotary_sin_->scalar_type() == q.scalar_type(),
                    "rotary_cos must have the same dtype as query");
    }
    Tensor mask;
    int n64 = 0;
    if (blockmask_.has_value()) {
        TORCH_CHECK(blockmask_->dim() == 4 && blockmask_->size(0) == batch && blockmask_->size(1) == Hk && blockmask_->size(2) == 1,
                    "topk_idx must have shape (batch_size, num_heads_k, 1, k)");
        mask = blockmask_->contiguous();
        n64 = static_cast<int>(mask.size(-1));
    }
    Tensor out = at::empty_like(q);
    Tensor lse = at::empty({batch, Hq, 1}, q.options().dtype(at::kFloat));
    const int splits = infllmv2_fwd_kvcache_num_splits(batch, Hk, static_cast<int>(num_splits));
    Tensor ws = bytes_on(q, infllmv2_fwd_kvcache_workspace_bytes(batch, Hk, splits));
    const int64_t qs[2] = {q.stride(0), q.stride(2)}, os[2] = {out.stride(0), out.stride(2)};
    const int64_t kcs[3] = {kcache.stride(0), kcache.stride(1), kcache.stride(2)};
    const int64_t vcs[3] = {vcache.stride(0), vcache.stride(1), vcache.stride(2)};
    int64_t kns[3] = {0, 0, 0}, vns[3] = {0, 0, 0};
    if (k_.has_value()) {
        for (int i = 0; i < 3; ++i) { kns[i] = k_->stride(i); vns[i] = v_->stride(i); }
    }
    auto fn = is_half(q) ? infllmv2_fwd_kvcache_f16 : infllmv2_fwd_kvcache;
    check_rc(fn(stream_of(q), q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), cptr(k_), cptr(v_),
                seqlens.defined() ? seqlens.data_ptr<int32_t>() : nullptr, out.data_ptr(), lse.data_ptr<float>(),
                mask.defined() ? reinterpret_cast<const uint64_t*>(mask.data_ptr()) : nullptr, ws.data_ptr(),
                static_cast<size_t>(ws.numel()), batch, seqlen_q, Hq, Hk, d, cap, seqlen_new, qs, kcs, vcs, kns, vns, os, n64,
                splits, static_cast<float>(softmax_scale), batch_idx.defined() ? batch_idx.data_ptr<int32_t>() : nullptr,
                leftpad.defined() ? leftpad.data_ptr<int32_t>() : nullptr,
                paged ? block_table_->data_ptr<int32_t>() : nullptr, table_stride, page, cptr(rotary_cos_), cptr(rotary_sin_),
                rotary_dim, is_rotary_interleaved ? 1 : 0), "fwd_kvcache");
    if (out_.has_value()) {
        out_->copy_(out);
        return {*out_, lse};
    }
    return {out, lse};
}

// ---- fixed-length batches: the packed entries with equal sequence lengths -----------------------------------------
Tensor packed(const Tensor& t, const char* name) {
    TORCH_CHECK(t.dim() == 4, name, " must have shape (batch_size, seqlen, num_heads, head_size)");
    return t.reshape({t.size(0) * t.size(1), t.size(2), t.size(3)});
}
Tensor equal_cu(int64_t batch, int64_t seqlen, const Tensor& like) {
    return at::arange(batch + 1, like.options().dtype(at::kInt)) * static_cast<int>(seqlen);
}

// mha_fwd (flash_api.cpp:349-517): dense attention over a fixed-length batch, q (b, sq, Hq, d), k/v (b, sk, Hk, d).
// Returns {out, softmax_lse (b, Hq, sq), p, rng_state}.
std::vector<Tensor> fwd(const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& out_, const OptTensor& alibi_slopes_,
                        double p_dropout, double softmax_scale, bool is_causal, int64_t window_size_left,
                        int64_t window_size_right, double softcap, bool return_softmax, const py::object& gen_) {
    TORCH_CHECK(q.dim() == 4 && k.dim() == 4, "q, k, v must have shape (batch_size, seqlen, num_heads, head_size)");
    const int64_t b = q.size(0), sq = q.size(1), Hq = q.size(2), d = q.size(3), sk = k.size(1);
    TORCH_CHECK(k.size(0) == b && v.sizes() == k.sizes(), "k and v must have shape (batch_size, seqlen_k, num_heads_k, head_size)");
    TORCH_CHECK(!out_.has_value() || out_->sizes() == q.sizes(), "out must have the shape of q");
    auto res = varlen_fwd(packed(q, "q"), packed(k, "k"), packed(v, "v"), std::nullopt, equal_cu(b, sq, q), equal_cu(b, sk, q),
                          std::nullopt, std::nullopt, std::nullopt, alibi_slopes_, sq, sk, p_dropout, softmax_scale, false,
                          is_causal, window_size_left, window_size_right, softcap, return_softmax, gen_, std::nullopt);
    Tensor out = res[0].view({b, sq, Hq, d});
    if (out_.has_value()) {
        out_->copy_(out);
        out = *out_;
    }
    Tensor lse = res[1].view({Hq, b, sq}).permute({1, 0, 2}).contiguous();
    return {out, lse, res[2], res[3]};
}

// mha_bwd (flash_api.cpp:1062-1276): gradients of `fwd`; softmax_lse (b, Hq, sq).  Returns {dq, dk, dv, softmax_d}.
std::vector<Tensor> bwd(const Tensor& dout, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& out,
                        const Tensor& softmax_lse, const OptTensor& dq_, const OptTensor& dk_, const OptTensor& dv_,
                        const OptTensor& alibi_slopes_, double p_dropout, double softmax_scale, bool is_causal,
                        int64_t window_size_left, int64_t window_size_right, double softcap, bool deterministic,
                        const py::object& gen_, const OptTensor& rng_state) {
    TORCH_CHECK(q.dim() == 4 && k.dim() == 4, "q, k, v must have shape (batch_size, seqlen, num_heads, head_size)");
    const int64_t b = q.size(0), sq = q.size(1), Hq = q.size(2), sk = k.size(1);
    TORCH_CHECK(softmax_lse.dim() == 3 && softmax_lse.size(0) == b && softmax_lse.size(1) == Hq && softmax_lse.size(2) == sq,
                "softmax_lse must have shape (batch_size, num_heads, seqlen_q)");
    Tensor lse = softmax_lse.permute({1, 0, 2}).reshape({Hq, b * sq}).contiguous();
    auto res = varlen_bwd(packed(dout, "dout"), packed(q, "q"), packed(k, "k"), packed(v, "v"), packed(out, "out"), lse,
                          std::nullopt, std::nullopt, std::nullopt, equal_cu(b, sq, q), equal_cu(b, sk, q), alibi_slopes_, sq, sk,
                          p_dropout, softmax_scale, false, is_causal, window_size_left, window_size_right, softcap,
                          deterministic, std::nullopt, gen_, rng_state);
    const OptTensor* given[3] = {&dq_, &dk_, &dv_};
    const Tensor* like[3] = {&q, &k, &v};
    std::vector<Tensor> grads;
    for (int i = 0; i < 3; ++i) {
        Tensor r = res[i].view(like[i]->sizes());
        if (given[i]->has_value()) {
            TORCH_CHECK((*given[i])->sizes() == like[i]->sizes(), "dq, dk, dv must have the shapes of q, k, v");
            (*given[i])->copy_(r);
            r = **given[i];
        }
        grads.push_back(r);
    }
    grads.push_back(res[3]);
    return grads;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "InfLLM-V2 sparse attention for MI355X: the reference's native module over libinfllmv2_hip.so";
    m.def("topk", &topk);
    m.def("get_probs", &get_probs);
    m.def("blockmask_to_uint64", &blockmask_to_uint64);
    m.def("topk_to_uint64", &topk_to_uint64);
    m.def("uint64_to_bool", &uint64_to_bool);
    m.def("max_pooling_1d", &max_pooling_1d);
    m.def("max_pooling_1d_varlen", &max_pooling_1d_varlen);
    m.def("fwd", &fwd, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out_"), py::arg("alibi_slopes_"), py::arg("p_dropout"),
          py::arg("softmax_scale"), py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"),
          py::arg("softcap"), py::arg("return_softmax"), py::arg("gen_") = py::none());
    m.def("varlen_fwd", &varlen_fwd, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out_"), py::arg("cu_seqlens_q"),
          py::arg("cu_seqlens_k"), py::arg("seqused_k"), py::arg("leftpad_k_"), py::arg("block_table_"), py::arg("alibi_slopes_"),
          py::arg("max_seqlen_q"), py::arg("max_seqlen_k"), py::arg("p_dropout"), py::arg("softmax_scale"), py::arg("zero_tensors"),
          py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"),
          py::arg("return_softmax"), py::arg("gen_") = py::none(), py::arg("blockmask_") = py::none());
    m.def("varlen_fwd_stage1", &varlen_fwd_stage1, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out_"), py::arg("cu_seqlens_q"),
          py::arg("cu_seqlens_k"), py::arg("cu_seqlens_v"), py::arg("seqused_k"), py::arg("leftpad_k_"), py::arg("block_table_"),
          py::arg("alibi_slopes_"), py::arg("max_seqlen_q"), py::arg("max_seqlen_k"), py::arg("p_dropout"), py::arg("softmax_scale"),
          py::arg("zero_tensors"), py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"),
          py::arg("softcap"), py::arg("return_softmax"), py::arg("gen_") = py::none());
    m.def("bwd", &bwd, py::arg("dout"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"), py::arg("softmax_lse"),
          py::arg("dq_"), py::arg("dk_"), py::arg("dv_"), py::arg("alibi_slopes_"), py::arg("p_dropout"), py::arg("softmax_scale"),
          py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"),
          py::arg("deterministic"), py::arg("gen_") = py::none(), py::arg("rng_state") = py::none());
    m.def("varlen_bwd", &varlen_bwd, py::arg("dout"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"), py::arg("softmax_lse"),
          py::arg("dq_"), py::arg("dk_"), py::arg("dv_"), py::arg("cu_seqlens_q"), py::arg("cu_seqlens_k"), py::arg("alibi_slopes_"),
          py::arg("max_seqlen_q"), py::arg("max_seqlen_k"), py::arg("p_dropout"), py::arg("softmax_scale"), py::arg("zero_tensors"),
          py::arg("is_causal"), py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"),
          py::arg("deterministic"), py::arg("col_blockmask_") = py::none(), py::arg("gen_") = py::none(),
          py::arg("rng_state") = py::none());
    m.def("fwd_kvcache", &fwd_kvcache, py::arg("q"), py::arg("kcache"), py::arg("vcache"), py::arg("k_"), py::arg("v_"),
          py::arg("seqlens_k_"), py::arg("rotary_cos_"), py::arg("rotary_sin_"), py::arg("cache_batch_idx_"), py::arg("leftpad_k_"),
          py::arg("block_table_"), py::arg("alibi_slopes_"), py::arg("out_"), py::arg("softmax_scale"), py::arg("is_causal"),
          py::arg("window_size_left"), py::arg("window_size_right"), py::arg("softcap"), py::arg("is_rotary_interleaved"),
          py::arg("num_splits"), py::arg("blockmask_") = py::none());
}
