// PyTorch-ROCm host layer: registers the reference's operator and class names in the
// `torch_dist_ext` namespace (src/register.cpp:4-15 of the reference) and forwards to the C ABI in
// tde_abi.h.  No kernels here; this file is compiled by the host compiler only.
//
// One GPU plays every rank: CommWorkspace owns N local allocations ("slots") where the reference
// maps N peers' comm buffers through HIP IPC (src/ops/all_reduce_fusion.cpp:107-141).
#include <ATen/ATen.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <unistd.h>

#include <cstring>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "tde_abi.h"

namespace {

using at::Tensor;

constexpr int64_t kHandleBytes = 64; // sizeof(hipIpcMemHandle_t), the size get_handle() returns in the reference
constexpr char kHandleMagic[8] = {'T', 'D', 'E', 'L', 'O', 'C', 'A', 'L'};

void check_status(int st, const char *what) {
    if (st == TDE_OK) return;
    if (st == TDE_EHIP) {
        TORCH_CHECK(false, what, ": ", tde_status_string(st), ", hipError ", tde_last_hip_error());
    }
    TORCH_CHECK(false, what, ": ", tde_status_string(st));
}

int32_t dtype_code(const Tensor &t) {
    switch (t.scalar_type()) {
    case at::kBFloat16: return TDE_BF16;
    case at::kHalf: return TDE_F16;
    case at::kFloat: return TDE_F32;
    case at::kDouble: return TDE_F64;
    default: TORCH_CHECK(false, "torch_dist_ext: unsupported dtype ", t.scalar_type(), " (bf16, fp16, fp32, fp64)");
    }
    return -1;
}

// Pointer tables handed out by CommWorkspace::get_workspace, keyed by their device address, with the size of
// the slots they point to.  The operators receive only the table tensor (the reference's signature), so this
// is how they learn how many bytes of each slot exist: a call whose rows do not fit is refused instead of
// reading past a slot.
std::mutex g_tables_mutex;
std::unordered_map<const void *, int64_t> g_table_slot_bytes;

void register_table(const void *table, int64_t slot_bytes) {
    const std::lock_guard<std::mutex> lock(g_tables_mutex);
    g_table_slot_bytes[table] = slot_bytes;
}

void unregister_table(const void *table) {
    const std::lock_guard<std::mutex> lock(g_tables_mutex);
    g_table_slot_bytes.erase(table);
}

// -1 if `table` was not handed out by a live CommWorkspace.
int64_t table_slot_bytes(const void *table) {
    const std::lock_guard<std::mutex> lock(g_tables_mutex);
    const auto it = g_table_slot_bytes.find(table);
    return it == g_table_slot_bytes.end() ? -1 : it->second;
}

void check_row_tensor(const Tensor &t, const Tensor &like, const char *name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(t.device() == like.device(), name, " is on a different device than allreduce_in");
    TORCH_CHECK(t.scalar_type() == like.scalar_type(), name, " dtype differs from allreduce_in");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.numel() == like.numel(), name, " numel differs from allreduce_in");
}

} // namespace

// Same constructor and method signatures as the reference class (src/ops/all_reduce_fusion.h:10-16).
class CommWorkspace : public torch::CustomClassHolder {
public:
    CommWorkspace(int64_t rank, int64_t world_size, int64_t nblocks, int64_t size_in_bytes)
        : rank_(rank), world_size_(world_size), nblocks_(nblocks), size_in_bytes_(size_in_bytes) {
        TORCH_CHECK(rank >= 0 && rank < world_size, "CommWorkspace: rank ", rank, " outside [0, ", world_size, ")");
        TORCH_CHECK(size_in_bytes > 0 && size_in_bytes % 16 == 0, "CommWorkspace: size_in_bytes must be a positive multiple of 16");
        device_ = c10::hip::current_device();
        TORCH_CHECK(nblocks >= 1 && nblocks <= 65536, "CommWorkspace: nblocks must be in [1, 65536]");
        check_status(tde_workspace_create((int32_t)world_size, (int32_t)nblocks, size_in_bytes, &ws_), "CommWorkspace");
    }

    ~CommWorkspace() override {
        if (table_.defined()) unregister_table(table_.data_ptr());
        tde_workspace_destroy(ws_);
    }

    // The reference returns the IPC handle of its allocation.  Nothing is exported here: the 64
    // bytes carry a tag, the process id, the rank and the address of slot `rank`.
    Tensor get_handle() {
        auto handle = at::zeros({kHandleBytes}, at::TensorOptions().dtype(at::kByte).device(at::kCPU));
        auto *p = handle.data_ptr<uint8_t>();
        std::memcpy(p, kHandleMagic, 8);
        const int64_t pid = (int64_t)getpid();
        const int64_t addr = (int64_t)reinterpret_cast<intptr_t>(tde_workspace_slot(ws_, (int32_t)rank_));
        std::memcpy(p + 8, &pid, 8);
        std::memcpy(p + 16, &rank_, 8);
        std::memcpy(p + 24, &addr, 8);
        return handle;
    }

    // The reference opens every peer's handle.  Peers are local slots here, so this only checks
    // the list: world_size handles of 64 bytes each, every one tagged as produced by get_handle().
    void open_handles(std::vector<Tensor> handles) {
        TORCH_CHECK((int64_t)handles.size() == world_size_, "open_handles: expected ", world_size_, " handles, got ",
                    handles.size());
        for (auto &h : handles) {
            TORCH_CHECK(h.device().is_cpu() && h.scalar_type() == at::kByte && h.numel() == kHandleBytes,
                        "open_handles: every handle must be a CPU uint8 tensor of 64 bytes");
            TORCH_CHECK(std::memcmp(h.data_ptr<uint8_t>(), kHandleMagic, 8) == 0,
                        "open_handles: handle was not produced by this library's get_handle()");
        }
        opened_ = true;
    }

    // uint8 device tensor of (3*world_size+5) pointers, layout of src/ops/all_reduce_fusion.cpp:159-169.
    // The table never changes after construction, so it is uploaded once and the same device
    // tensor is handed out afterwards (the reference rebuilds and copies it on every call,
    // src/ops/all_reduce_fusion.cpp:159-173): no host-to-device copy in steady state, which also
    // keeps the call legal while a HIP graph is being captured.
    Tensor get_workspace(const Tensor &ref) {
        TORCH_CHECK(ref.is_cuda() && ref.device().index() == device_,
                    "get_workspace: ref must live on the workspace's GPU (device ", device_, "): the table holds that device's pointers");
        if (table_.defined()) return table_;
        const int64_t entries = 3 * world_size_ + 5;
        auto host = at::empty({entries * (int64_t)sizeof(void *)}, at::TensorOptions().dtype(at::kByte).device(at::kCPU));
        check_status(tde_workspace_fill_table(ws_, reinterpret_cast<void **>(host.data_ptr()), (int32_t)entries),
                     "get_workspace");
        table_ = host.to(ref.device());
        register_table(table_.data_ptr(), size_in_bytes_);
        return table_;
    }

    // ---- emulation-only additions (no counterpart in the reference) -----------------------------
    // A tensor shaped and typed like `ref` that aliases slot r: what rank r's kernel would have
    // written into this rank's view of its comm buffer.
    Tensor peer_partial(int64_t r, const Tensor &ref) {
        TORCH_CHECK(r >= 0 && r < world_size_, "peer_partial: rank ", r, " outside [0, ", world_size_, ")");
        const int64_t bytes = ref.numel() * (int64_t)ref.element_size();
        TORCH_CHECK(bytes <= size_in_bytes_, "peer_partial: ", bytes, " bytes exceed the slot size ", size_in_bytes_);
        TORCH_CHECK(ref.is_cuda() && ref.device().index() == device_, "peer_partial: ref must live on the workspace's GPU");
        return alias(tde_workspace_slot(ws_, (int32_t)r), ref);
    }

    void set_peer_partial(int64_t r, const Tensor &src) {
        Tensor dst = peer_partial(r, src);
        dst.copy_(src, /*non_blocking=*/true);
    }

    // Stage half of slot `rank` (the gathered region of the reference's two-shot buffer).
    Tensor stage(const Tensor &ref) {
        const int64_t bytes = ref.numel() * (int64_t)ref.element_size();
        TORCH_CHECK(bytes <= size_in_bytes_, "stage: ", bytes, " bytes exceed the slot size ", size_in_bytes_);
        return alias(tde_workspace_stage(ws_, (int32_t)rank_), ref);
    }

    // Makes this workspace the one torch_dist_ext::get_workspace hands out (the reference keeps it in the Python
    // package's global `comm`, torch_dist_ext/__init__.py:37-46; the operator is registered in C++ here, so the
    // current workspace is kept here as well).  The previous one is released.
    void make_current();

    int64_t rank() const { return rank_; }
    int64_t world_size() const { return world_size_; }
    int64_t size_in_bytes() const { return size_in_bytes_; }

private:
    // A tensor like `ref` over workspace memory.  It holds a reference to this object, so the memory
    // outlives every such tensor.
    Tensor alias(void *ptr, const Tensor &ref) {
        auto self = c10::intrusive_ptr<CommWorkspace>::unsafe_reclaim_from_nonowning(this);
        return at::from_blob(ptr, ref.sizes(), [self](void *) {}, ref.options());
    }

    int64_t rank_, world_size_, nblocks_, size_in_bytes_;
    int device_ = 0;
    bool opened_ = false;
    tde_workspace *ws_ = nullptr;
    Tensor table_;
};

namespace {

std::mutex g_current_mutex;
// Never destroyed: releasing device memory during static destruction would run after the HIP runtime has gone.
c10::intrusive_ptr<CommWorkspace> *g_current = new c10::intrusive_ptr<CommWorkspace>();

} // namespace

void CommWorkspace::make_current() {
    auto self = c10::intrusive_ptr<CommWorkspace>::unsafe_reclaim_from_nonowning(this);
    const std::lock_guard<std::mutex> lock(g_current_mutex);
    *g_current = std::move(self);
}

namespace {

// torch_dist_ext::get_workspace (reference: a Python custom_op over the package's global, torch_dist_ext/__init__.py:49-53).
Tensor get_workspace_op(const Tensor &ref) {
    c10::intrusive_ptr<CommWorkspace> cur;
    {
        const std::lock_guard<std::mutex> lock(g_current_mutex);
        cur = *g_current;
    }
    TORCH_CHECK(cur.defined(), "torch_dist_ext::get_workspace: setup_env has not been called");
    return cur->get_workspace(ref);
}

struct Call {
    tde_problem p{};
    tde_buffers b{};
};

void fill_common(Call &c, int64_t rank, int64_t nranks, const Tensor &allreduce_in, const Tensor &residual_in,
                 const Tensor &rms_gamma, const Tensor &residual_out, double eps) {
    TORCH_CHECK(allreduce_in.is_cuda(), "allreduce_in must be a GPU tensor");
    TORCH_CHECK(allreduce_in.dim() >= 1 && allreduce_in.is_contiguous(), "allreduce_in must be contiguous");
    check_row_tensor(residual_in, allreduce_in, "residual_in");
    check_row_tensor(residual_out, allreduce_in, "residual_out");
    TORCH_CHECK(rms_gamma.is_cuda() && rms_gamma.is_contiguous() && rms_gamma.scalar_type() == allreduce_in.scalar_type() &&
                    rms_gamma.numel() == allreduce_in.size(-1),
                "rms_gamma must be a contiguous GPU tensor of allreduce_in's dtype with hidden elements");
    c.p.dtype = dtype_code(allreduce_in);
    c.p.nranks = (int32_t)nranks;
    c.p.rank = (int32_t)rank;
    c.p.hidden = allreduce_in.size(-1);
    c.p.tokens = c.p.hidden > 0 ? allreduce_in.numel() / c.p.hidden : 0;
    c.p.eps = (float)eps;
    c.b.residual_in = residual_in.data_ptr();
    c.b.residual_out = residual_out.data_ptr();
    c.b.gamma = rms_gamma.data_ptr();
}

void fill_quant(Call &c, int64_t quant_mode, const Tensor &like, const c10::optional<Tensor> &norm_out,
                const c10::optional<Tensor> &q_out, const c10::optional<Tensor> &scale_out, double static_scale = 0.0) {
    c.p.quant = (int32_t)quant_mode;
    c.p.static_scale = (float)static_scale;
    if (norm_out.has_value() && norm_out->defined()) {
        check_row_tensor(*norm_out, like, "norm_out");
        c.b.norm_out = norm_out->data_ptr();
        c.p.write_norm = 1;
    }
    if (quant_mode == TDE_QUANT_FP8_STATIC) {
        TORCH_CHECK(q_out.has_value() && q_out->defined(), "static fp8 quant needs q_out");
        TORCH_CHECK(q_out->is_cuda() && q_out->is_contiguous() && q_out->element_size() == 1 && q_out->numel() == like.numel(),
                    "q_out must be a contiguous 1-byte GPU tensor with allreduce_in's numel");
        c.b.q_out = q_out->data_ptr();
    } else if (quant_mode != TDE_QUANT_NONE) {
        TORCH_CHECK(q_out.has_value() && scale_out.has_value() && q_out->defined() && scale_out->defined(),
                    "dynamic quant modes need q_out and scale_out");
        TORCH_CHECK(q_out->is_cuda() && q_out->is_contiguous() && q_out->element_size() == 1 && q_out->numel() == like.numel(),
                    "q_out must be a contiguous 1-byte GPU tensor with allreduce_in's numel");
        const int64_t tokens = c.p.tokens;
        const int64_t want = (quant_mode == TDE_QUANT_FP8_GROUP) ? tokens * (c.p.hidden / TDE_QUANT_GROUP) : tokens;
        TORCH_CHECK(scale_out->is_cuda() && scale_out->is_contiguous() && scale_out->scalar_type() == at::kFloat &&
                        scale_out->numel() == want,
                    "scale_out must be a contiguous fp32 GPU tensor with ", want, " elements");
        c.b.q_out = q_out->data_ptr();
        c.b.scale_out = scale_out->data_ptr<float>();
    } else {
        TORCH_CHECK(c.b.norm_out != nullptr, "norm_out is required without quant");
    }
}

void run(Call &c, const Tensor &on) {
    const c10::hip::HIPGuard guard(on.device().index());
    hipStream_t stream = c10::hip::getCurrentHIPStream(on.device().index()).stream();
    check_status(tde_reduce_rms(&c.p, &c.b, stream), "torch_dist_ext");
}

// Points the call at the workspace's slots, with the caller's own partial read straight from allreduce_in.
void use_table(Call &c, int64_t rank, int64_t nranks, const Tensor &allreduce_in, const Tensor &workspace) {
    TORCH_CHECK(nranks == 2 || nranks == 4 || nranks == 8, "torch_dist_ext: ", tde_status_string(TDE_ENRANKS));
    TORCH_CHECK(workspace.is_cuda() && workspace.scalar_type() == at::kByte && workspace.is_contiguous() &&
                    workspace.numel() >= (3 * nranks + 5) * (int64_t)sizeof(void *),
                "workspace must be the uint8 GPU pointer table returned by get_workspace for this world size");
    TORCH_CHECK(rank >= 0 && rank < nranks && nranks <= TDE_MAX_RANKS, "rank/nranks out of range");
    const int64_t slot_bytes = table_slot_bytes(workspace.data_ptr());
    TORCH_CHECK(slot_bytes >= 0, "workspace is not a pointer table handed out by a live CommWorkspace's get_workspace "
                                 "(pass that tensor itself, not a copy)");
    TORCH_CHECK(allreduce_in.is_cuda() && allreduce_in.device() == workspace.device(),
                "allreduce_in must live on the workspace's GPU: the pointer table holds that device's addresses");
    const int64_t bytes = allreduce_in.numel() * (int64_t)allreduce_in.element_size();
    TORCH_CHECK(bytes <= slot_bytes, "allreduce_in has ", bytes, " bytes but the workspace slots hold ", slot_bytes,
                "; create the workspace (setup_env) with a larger size");
    c.b.partial_table = reinterpret_cast<const void *const *>(workspace.data_ptr());
    c.b.partial[rank] = allreduce_in.data_ptr();
}

// Reference entry point, verbatim signature (src/ops/all_reduce_fusion.h:42-43).  `workspace` is
// the device pointer table from CommWorkspace::get_workspace; its first nranks entries are the
// slots.  The caller's own partial is read straight from allreduce_in (the reference first copies
// it into its comm buffer, impl.h:354-360, 434-443).
void allreduce_rms_fusion(int64_t rank, int64_t nranks, Tensor &allreduce_in, Tensor &residual_in, Tensor &rms_gamma,
                          Tensor &residual_out, Tensor &norm_out, double eps, Tensor &workspace) {
    Call c;
    fill_common(c, rank, nranks, allreduce_in, residual_in, rms_gamma, residual_out, eps);
    fill_quant(c, TDE_QUANT_NONE, allreduce_in, norm_out, c10::nullopt, c10::nullopt);
    use_table(c, rank, nranks, allreduce_in, workspace);
    run(c, allreduce_in);
}

// Quantizing variant behind the same workspace protocol.
void allreduce_rms_quant_fusion(int64_t rank, int64_t nranks, Tensor &allreduce_in, Tensor &residual_in, Tensor &rms_gamma,
                                Tensor &residual_out, c10::optional<Tensor> norm_out, Tensor &q_out,
                                c10::optional<Tensor> scale_out, double eps, Tensor &workspace, int64_t quant_mode,
                                double static_scale) {
    Call c;
    fill_common(c, rank, nranks, allreduce_in, residual_in, rms_gamma, residual_out, eps);
    fill_quant(c, quant_mode, allreduce_in, norm_out, q_out, scale_out, static_scale);
    use_table(c, rank, nranks, allreduce_in, workspace);
    run(c, allreduce_in);
}

// Functional form, the operator the reference's package defines in Python (torch_dist_ext/__init__.py:64-73:
// a torch.library.custom_op that allocates norm_out and residual_out and calls allreduce_rms_fusion).  Registered
// here instead, same name and schema: a Python custom_op costs 12 us of host time per call, which is more than
// the kernel takes at decode sizes.  The hidden_dim <= 8192 assertion of the reference (:68) is a check here.
std::tuple<Tensor, Tensor> allreduce_rms(int64_t rank, int64_t nranks, const Tensor &allreduce_in, const Tensor &residual_in,
                                         const Tensor &rms_gamma, double eps, const Tensor &workspace) {
    TORCH_CHECK(allreduce_in.dim() >= 1 && allreduce_in.size(-1) <= 8192, "allreduce_rms: hidden_dim <= 8192 expected");
    Tensor norm_out = at::empty_like(allreduce_in);
    Tensor residual_out = at::empty_like(residual_in);
    Call c;
    fill_common(c, rank, nranks, allreduce_in, residual_in, rms_gamma, residual_out, eps);
    c.p.quant = TDE_QUANT_NONE;
    c.b.norm_out = norm_out.data_ptr();
    c.p.write_norm = 1;
    use_table(c, rank, nranks, allreduce_in, workspace);
    run(c, allreduce_in);
    return {norm_out, residual_out};
}

// Shapes and dtypes only: what tracing (fake tensors, torch.compile) sees.
std::tuple<Tensor, Tensor> allreduce_rms_meta(int64_t, int64_t, const Tensor &allreduce_in, const Tensor &residual_in,
                                              const Tensor &, double, const Tensor &) {
    return {at::empty_like(allreduce_in), at::empty_like(residual_in)};
}

struct QuantOutputs {
    Tensor q, scale, residual_out, norm_out;
};

// Output tensors of the quantizing operator: codes (e4m3 or int8) shaped like the input, scales [..., 1] per row or
// [..., hidden/128] per group (no elements with a static scale), residual_out, and norm_out (no elements unless asked for).
QuantOutputs quant_outputs(const Tensor &allreduce_in, const Tensor &residual_in, int64_t quant_mode, bool write_norm) {
    TORCH_CHECK(allreduce_in.dim() >= 1 && allreduce_in.size(-1) <= 8192, "allreduce_rms_quant: hidden_dim <= 8192 expected");
    TORCH_CHECK(quant_mode == TDE_QUANT_FP8_TOKEN || quant_mode == TDE_QUANT_FP8_GROUP || quant_mode == TDE_QUANT_INT8_TOKEN ||
                    quant_mode == TDE_QUANT_FP8_STATIC,
                "allreduce_rms_quant: quant_mode must be one of the quantizing modes (1..4)");
    QuantOutputs o;
    const auto q_dtype = quant_mode == TDE_QUANT_INT8_TOKEN ? at::kChar : at::kFloat8_e4m3fn;
    o.q = at::empty(allreduce_in.sizes(), allreduce_in.options().dtype(q_dtype));
    std::vector<int64_t> scale_shape(allreduce_in.sizes().begin(), allreduce_in.sizes().end() - 1);
    if (quant_mode == TDE_QUANT_FP8_GROUP) scale_shape.push_back(allreduce_in.size(-1) / TDE_QUANT_GROUP);
    if (quant_mode == TDE_QUANT_FP8_STATIC) scale_shape.assign(1, 0);
    o.scale = at::empty(scale_shape, allreduce_in.options().dtype(at::kFloat));
    o.residual_out = at::empty_like(residual_in);
    o.norm_out = write_norm ? at::empty_like(allreduce_in) : at::empty({0}, allreduce_in.options());
    return o;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> allreduce_rms_quant(int64_t rank, int64_t nranks, const Tensor &allreduce_in,
                                                               const Tensor &residual_in, const Tensor &rms_gamma, double eps,
                                                               const Tensor &workspace, int64_t quant_mode, bool write_norm,
                                                               double static_scale) {
    QuantOutputs o = quant_outputs(allreduce_in, residual_in, quant_mode, write_norm);
    Call c;
    fill_common(c, rank, nranks, allreduce_in, residual_in, rms_gamma, o.residual_out, eps);
    fill_quant(c, quant_mode, allreduce_in, write_norm ? c10::optional<Tensor>(o.norm_out) : c10::nullopt, o.q,
               quant_mode == TDE_QUANT_FP8_STATIC ? c10::nullopt : c10::optional<Tensor>(o.scale), static_scale);
    use_table(c, rank, nranks, allreduce_in, workspace);
    run(c, allreduce_in);
    return {o.q, o.scale, o.residual_out, o.norm_out};
}

std::tuple<Tensor, Tensor, Tensor, Tensor> allreduce_rms_quant_meta(int64_t, int64_t, const Tensor &allreduce_in,
                                                                    const Tensor &residual_in, const Tensor &, double, const Tensor &,
                                                                    int64_t quant_mode, bool write_norm, double) {
    QuantOutputs o = quant_outputs(allreduce_in, residual_in, quant_mode, write_norm);
    return {o.q, o.scale, o.residual_out, o.norm_out};
}

// The same stage with the N partials given directly as N tensors (no workspace object).
void reduce_rms_local(std::vector<Tensor> partials, Tensor &residual_in, Tensor &rms_gamma, Tensor &residual_out,
                      c10::optional<Tensor> norm_out, c10::optional<Tensor> q_out, c10::optional<Tensor> scale_out,
                      double eps, int64_t quant_mode, int64_t algo, c10::optional<Tensor> stage, double static_scale) {
    TORCH_CHECK(!partials.empty() && partials.size() <= TDE_MAX_RANKS, "reduce_rms_local: 2, 4 or 8 partials expected");
    Call c;
    fill_common(c, 0, (int64_t)partials.size(), partials[0], residual_in, rms_gamma, residual_out, eps);
    fill_quant(c, quant_mode, partials[0], norm_out, q_out, scale_out, static_scale);
    for (size_t r = 0; r < partials.size(); ++r) {
        check_row_tensor(partials[r], partials[0], "partial");
        c.b.partial[r] = partials[r].data_ptr();
    }
    c.p.algo = (int32_t)algo;
    if (stage.has_value() && stage->defined()) {
        check_row_tensor(*stage, partials[0], "stage");
        c.b.stage = stage->data_ptr();
    }
    run(c, partials[0]);
}

} // namespace

TORCH_LIBRARY(torch_dist_ext, m) {
    m.class_<CommWorkspace>("CommWorkspace")
        .def(torch::init<int64_t, int64_t, int64_t, int64_t>())
        .def("get_handle", &CommWorkspace::get_handle)
        .def("open_handles", &CommWorkspace::open_handles)
        .def("get_workspace", &CommWorkspace::get_workspace)
        .def("peer_partial", &CommWorkspace::peer_partial)
        .def("set_peer_partial", &CommWorkspace::set_peer_partial)
        .def("stage", &CommWorkspace::stage)
        .def("make_current", &CommWorkspace::make_current)
        .def("rank", &CommWorkspace::rank)
        .def("world_size", &CommWorkspace::world_size)
        .def("size_in_bytes", &CommWorkspace::size_in_bytes);
    m.def("allreduce_rms_fusion(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, "
          "Tensor residual_out, Tensor norm_out, float eps, Tensor workspace) -> ()");
    m.def("allreduce_rms_quant_fusion(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, "
          "Tensor residual_out, Tensor? norm_out, Tensor q_out, Tensor? scale_out, float eps, Tensor workspace, "
          "int quant_mode, float static_scale=0.0) -> ()");
    m.def("get_workspace(Tensor ref) -> Tensor");
    m.def("allreduce_rms(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, float eps, "
          "Tensor workspace) -> (Tensor, Tensor)");
    m.def("allreduce_rms_quant(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, Tensor rms_gamma, float eps, "
          "Tensor workspace, SymInt quant_mode, bool write_norm, float static_scale=0.0) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("reduce_rms_local(Tensor[] partials, Tensor residual_in, Tensor rms_gamma, Tensor residual_out, "
          "Tensor? norm_out, Tensor? q_out, Tensor? scale_out, float eps, int quant_mode, int algo, Tensor? stage, "
          "float static_scale=0.0) -> ()");
}

TORCH_LIBRARY_IMPL(torch_dist_ext, CUDA, m) {
    m.impl("allreduce_rms_fusion", &allreduce_rms_fusion);
    m.impl("allreduce_rms_quant_fusion", &allreduce_rms_quant_fusion);
    m.impl("reduce_rms_local", &reduce_rms_local);
    m.impl("allreduce_rms", &allreduce_rms);
    m.impl("allreduce_rms_quant", &allreduce_rms_quant);
    m.impl("get_workspace", &get_workspace_op);
}

TORCH_LIBRARY_IMPL(torch_dist_ext, Meta, m) {
    m.impl("allreduce_rms", &allreduce_rms_meta);
    m.impl("allreduce_rms_quant", &allreduce_rms_quant_meta);
}
