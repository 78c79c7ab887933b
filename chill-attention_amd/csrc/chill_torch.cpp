// Eager-mode operator of the Python package, registered from C++: chill_attention_amd::attention.
//
// The reference registers its operators from Python (chill.py:60-80, torch.library.custom_op) and so does
// this package for torch.compile; a call through that layer costs ~30 us forward and ~130 us
// forward + backward on the host, more than the kernels of a short sequence take.  This file is the
// same adapter pair (chill.py:82-216 forward, 218-446 backward) and the same autograd formula
// (chill.py:448-474) in C++: it allocates the outputs with ATen and hands raw pointers and strides to
// the C ABI of include/chill_attention.h.  It links against no kernel library: the caller passes the
// addresses of its entry points (the stock library's, or those of the library built around a
// user-written mask), so one operator serves every mask class.
//
// The Python caller validates its inputs (chill.py, _check_inputs) with the reference's messages; the checks
// that keep a direct call of the operator from crashing the process (devices, dtypes, shapes, the table of
// entry points) are repeated here.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <cstring>
#include <deque>
#include <mutex>

#include "../../include/chill_attention.h"

namespace {

// The entry points of one kernel library.  The Python side (ctypes) fills a table per library and registers
// it once through chill_torch_register_entry_points; the operator takes the small handle that call returns,
// never an address.
constexpr uint64_t kEntryPointsMagic = 0x4350454c4c494843ull;  // "CHILLEPC"
struct EntryPoints {
    uint64_t magic;        // kEntryPointsMagic
    uint32_t abi_version;  // CHILL_ABI_VERSION of the header the table was filled against
    uint32_t bytes;        // sizeof(EntryPoints)
    decltype(&chill_fwd) fwd;
    decltype(&chill_bwd_dq_delta) dq_delta;
    decltype(&chill_bwd_dkdv) dkdv;
    decltype(&chill_status_string) status_string;
};

std::mutex g_tables_mutex;
std::deque<EntryPoints> g_tables;  // (a deque: registered tables never move)

const EntryPoints* table_of(int64_t handle) {
    std::lock_guard<std::mutex> lock(g_tables_mutex);
    TORCH_CHECK(handle >= 0 && handle < (int64_t)g_tables.size(), "chill_attention: ", handle,
                " is not a handle of chill_torch_register_entry_points (", g_tables.size(), " registered)");
    return &g_tables[(size_t)handle];
}

int32_t dtype_code(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kFloat: return CHILL_F32;
        case at::kHalf: return CHILL_F16;
        case at::kBFloat16: return CHILL_BF16;
        default: TORCH_CHECK(false, "chill_attention: q, k, v must be fp32, fp16 or bf16");
    }
}

// A view the kernels can address (unit inner stride, 16-byte aligned base and outer strides), copying
// only if the tensor does not already qualify.
at::Tensor kernel_view(const at::Tensor& t) {
    const int64_t es = t.element_size();
    bool ok = t.stride(-1) == 1 && reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0;
    for (int64_t i = 0; ok && i + 1 < t.dim(); i++) ok = t.stride(i) >= 0 && (t.stride(i) * es) % 16 == 0;
    return ok ? t : t.contiguous();
}

ChillTensor4 tensor4(const at::Tensor& t) {
    ChillTensor4 r;
    r.ptr = t.data_ptr();
    for (int i = 0; i < 4; i++) r.stride[i] = t.stride(i);
    return r;
}

ChillMaskDesc mask_desc(int64_t mask_id, at::IntArrayRef args) {
    TORCH_CHECK(args.size() <= 4, "chill_attention: a mask takes at most four arguments");
    ChillMaskDesc d;
    d.id = (int32_t)mask_id;
    d.nargs = (int32_t)args.size();
    for (int i = 0; i < 4; i++) d.args[i] = i < (int)args.size() ? args[i] : 0;
    return d;
}

void check(const EntryPoints* ep, const char* what, int status) {
    TORCH_CHECK(status >= 0, what, " failed with status ", status, ": ", ep->status_string(status));
}

// what the kernels assume of their operands and the C ABI cannot see from a raw pointer
void check_operands(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const c10::optional<at::Tensor>& lens) {
    TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), "chill_attention: q, k, v must be GPU tensors");
    TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "chill_attention: q, k, v must be on one device");
    TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "chill_attention: q, k, v must be [B, H, T, D]");
    TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(),
                "chill_attention: q, k, v must have one dtype");
    TORCH_CHECK(k.sizes() == v.sizes() && k.size(0) == q.size(0) && k.size(2) == q.size(2) && k.size(3) == q.size(3),
                "chill_attention: k, v must be [B, H_kv, T, D] for q of [B, H, T, D]");
    TORCH_CHECK(k.size(1) > 0 && q.size(1) % k.size(1) == 0, "chill_attention: H must be a multiple of H_kv");
    if (lens.has_value() && lens->defined())
        TORCH_CHECK(lens->device() == q.device() && lens->scalar_type() == at::kInt && lens->dim() == 1 &&
                        lens->size(0) == q.size(0),
                    "chill_attention: lens must be an int32 tensor of [B] on the device of q");
}

std::tuple<at::Tensor, at::Tensor> forward_impl(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                                const c10::optional<at::Tensor>& lens, int64_t entry_points,
                                                int64_t mask_id, at::IntArrayRef mask_args, double sm_scale,
                                                bool return_lse) {
    const EntryPoints* ep = table_of(entry_points);
    check_operands(q, k, v, lens);
    c10::DeviceGuard guard(q.device());
    const at::Tensor qv = kernel_view(q), kv = kernel_view(k), vv = kernel_view(v);
    // the kernel writes every row (zeros where nothing attends), so no zero fill is needed
    at::Tensor o = at::empty_like(q, q.options(), at::MemoryFormat::Contiguous);
    at::Tensor lse = return_lse ? at::empty({q.size(0), q.size(1), q.size(2)}, q.options().dtype(at::kFloat))
                                : at::empty({0}, q.options().dtype(at::kFloat));
    const ChillTensor4 tq = tensor4(qv), tk = tensor4(kv), tv = tensor4(vv), to = tensor4(o);
    const ChillMaskDesc desc = mask_desc(mask_id, mask_args);
    const int64_t lse_stride[3] = {return_lse ? lse.stride(0) : 0, return_lse ? lse.stride(1) : 0, return_lse ? lse.stride(2) : 0};
    const bool has_lens = lens.has_value() && lens->defined();
    check(ep, "chill_fwd",
          ep->fwd(&tq, &tk, &tv, &to, return_lse ? lse.data_ptr<float>() : nullptr, return_lse ? lse_stride : nullptr,
                  has_lens ? lens->data_ptr<int32_t>() : nullptr, has_lens ? lens->stride(0) : 0, (int32_t)q.size(0),
                  (int32_t)q.size(1), (int32_t)k.size(1), (int32_t)q.size(2), (int32_t)q.size(3), dtype_code(q),
                  (float)sm_scale, &desc, c10::hip::getCurrentHIPStream(q.device().index()).stream()));
    return {o, lse};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> backward_impl(const at::Tensor& q, const at::Tensor& k,
                                                             const at::Tensor& v, const c10::optional<at::Tensor>& lens,
                                                             const at::Tensor& o, const at::Tensor& lse_in,
                                                             const at::Tensor& d_o, int64_t entry_points, int64_t mask_id,
                                                             at::IntArrayRef mask_args, double sm_scale) {
    const EntryPoints* ep = table_of(entry_points);
    check_operands(q, k, v, lens);
    TORCH_CHECK(o.sizes() == q.sizes() && d_o.sizes() == q.sizes() && o.device() == q.device() && d_o.device() == q.device() &&
                    o.scalar_type() == q.scalar_type(),
                "chill_attention: o and its gradient must match q");
    TORCH_CHECK(lse_in.device() == q.device() && lse_in.scalar_type() == at::kFloat && lse_in.dim() == 3 &&
                    lse_in.size(0) == q.size(0) && lse_in.size(1) == q.size(1) && lse_in.size(2) == q.size(2),
                "chill_attention: the saved LSE must be fp32 [B, H, T]");
    c10::DeviceGuard guard(q.device());
    const at::Tensor qv = kernel_view(q), kv = kernel_view(k), vv = kernel_view(v), ov = kernel_view(o);
    const at::Tensor dov = kernel_view(d_o.scalar_type() == q.scalar_type() ? d_o : d_o.to(q.scalar_type()));
    const at::Tensor lse = lse_in.contiguous();
    at::Tensor delta = at::empty({q.size(0), q.size(1), q.size(2)}, q.options().dtype(at::kFloat));
    at::Tensor dq = at::empty_like(q, q.options(), at::MemoryFormat::Contiguous);
    at::Tensor dk = at::empty_like(k, k.options(), at::MemoryFormat::Contiguous);
    at::Tensor dv = at::empty_like(v, v.options(), at::MemoryFormat::Contiguous);
    const ChillTensor4 tq = tensor4(qv), tk = tensor4(kv), tv = tensor4(vv), to = tensor4(ov), tdo = tensor4(dov);
    const ChillTensor4 tdq = tensor4(dq), tdk = tensor4(dk), tdv = tensor4(dv);
    const ChillMaskDesc desc = mask_desc(mask_id, mask_args);
    const int64_t lse_stride[3] = {lse.stride(0), lse.stride(1), lse.stride(2)};
    const int64_t delta_stride[3] = {delta.stride(0), delta.stride(1), delta.stride(2)};
    const bool has_lens = lens.has_value() && lens->defined();
    const int32_t* lens_ptr = has_lens ? lens->data_ptr<int32_t>() : nullptr;
    const int64_t lens_stride = has_lens ? lens->stride(0) : 0;
    const int32_t B = (int32_t)q.size(0), H = (int32_t)q.size(1), H_kv = (int32_t)k.size(1), T = (int32_t)q.size(2),
                  D = (int32_t)q.size(3), dtype = dtype_code(q);
    void* stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    // dQ first: it computes delta of its rows on the way and leaves it for dK/dV
    check(ep, "chill_bwd_dq_delta",
          ep->dq_delta(&tq, &tk, &tv, &to, &tdo, &tdq, lse.data_ptr<float>(), lse_stride, delta.data_ptr<float>(),
                       delta_stride, lens_ptr, lens_stride, B, H, H_kv, T, D, dtype, (float)sm_scale, &desc, stream));
    check(ep, "chill_bwd_dkdv",
          ep->dkdv(&tq, &tk, &tv, &tdo, &tdk, &tdv, lse.data_ptr<float>(), lse_stride, delta.data_ptr<float>(),
                   delta_stride, lens_ptr, lens_stride, B, H, H_kv, T, D, dtype, (float)sm_scale, &desc, stream));
    return {dq, dk, dv};
}

// The autograd formula of chill.py:448-474: LSE is not differentiated; one gradient per tensor input.
class Attention : public torch::autograd::Function<Attention> {
  public:
    static torch::autograd::variable_list forward(torch::autograd::AutogradContext* ctx, const at::Tensor& q,
                                                  const at::Tensor& k, const at::Tensor& v,
                                                  const c10::optional<at::Tensor>& lens, int64_t entry_points,
                                                  int64_t mask_id, std::vector<int64_t> mask_args, double sm_scale,
                                                  bool return_lse) {
        at::AutoDispatchBelowADInplaceOrView below;
        const bool needs_grad = q.requires_grad() || k.requires_grad() || v.requires_grad();
        auto [o, lse] = forward_impl(q, k, v, lens, entry_points, mask_id, mask_args, sm_scale, return_lse || needs_grad);
        if (needs_grad) {
            ctx->save_for_backward({q, k, v, o, lse, lens.has_value() && lens->defined() ? *lens : at::Tensor()});
            ctx->saved_data["entry_points"] = entry_points;
            ctx->saved_data["mask_id"] = mask_id;
            ctx->saved_data["mask_args"] = mask_args;
            ctx->saved_data["sm_scale"] = sm_scale;
        }
        ctx->mark_non_differentiable({lse});
        return {o, lse};
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const c10::optional<at::Tensor> lens = saved[5].defined() ? c10::optional<at::Tensor>(saved[5]) : c10::nullopt;
        auto [dq, dk, dv] = backward_impl(saved[0], saved[1], saved[2], lens, saved[3], saved[4], grads[0],
                                          ctx->saved_data["entry_points"].toInt(), ctx->saved_data["mask_id"].toInt(),
                                          ctx->saved_data["mask_args"].toIntVector(), ctx->saved_data["sm_scale"].toDouble());
        return {dq, dk, dv, at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor(), at::Tensor()};
    }
};

std::tuple<at::Tensor, at::Tensor> attention_autograd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                                      const c10::optional<at::Tensor>& lens, int64_t entry_points,
                                                      int64_t mask_id, at::IntArrayRef mask_args, double sm_scale,
                                                      bool return_lse) {
    // where autograd is switched off (torch.no_grad) nothing is recorded: no LSE is computed for a backward that
    // cannot come, and nothing is saved
    if (!at::GradMode::is_enabled() || !(q.requires_grad() || k.requires_grad() || v.requires_grad())) {
        at::AutoDispatchBelowADInplaceOrView below;
        return forward_impl(q, k, v, lens, entry_points, mask_id, mask_args, sm_scale, return_lse);
    }
    auto out = Attention::apply(q, k, v, lens, entry_points, mask_id, mask_args.vec(), sm_scale, return_lse);
    return {out[0], out[1]};
}

}  // namespace

// Registers a table of entry points; returns its handle (>= 0), or -1 if the table is not one (wrong magic or
// size) and -2 if it was filled against another version of the C ABI.
extern "C" int64_t chill_torch_register_entry_points(const void* table) {
    if (table == nullptr) return -1;
    EntryPoints t;
    std::memcpy(&t, table, sizeof(uint64_t) + 2 * sizeof(uint32_t));
    if (t.magic != kEntryPointsMagic || t.bytes != sizeof(EntryPoints)) return -1;
    if (t.abi_version != CHILL_ABI_VERSION) return -2;
    std::memcpy(&t, table, sizeof(EntryPoints));
    if (!t.fwd || !t.dq_delta || !t.dkdv || !t.status_string) return -1;
    std::lock_guard<std::mutex> lock(g_tables_mutex);
    g_tables.push_back(t);
    return (int64_t)g_tables.size() - 1;
}

TORCH_LIBRARY(chill_attention_amd, m) {
    m.def(
        "attention(Tensor q, Tensor k, Tensor v, Tensor? lens, int entry_points, int mask_id, int[] mask_args, "
        "float sm_scale, bool return_lse) -> (Tensor, Tensor)");
}

// tensors that autograd does not track (inference mode) reach the device kernel directly
TORCH_LIBRARY_IMPL(chill_attention_amd, CUDA, m) { m.impl("attention", &forward_impl); }
TORCH_LIBRARY_IMPL(chill_attention_amd, Autograd, m) { m.impl("attention", &attention_autograd); }
