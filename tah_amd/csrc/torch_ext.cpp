// PyTorch-ROCm extension over the C ABI of include/tah_duo.h.
//
// Python hands tensors to the functions below; each one checks shapes, dtypes and devices, allocates the
// outputs through torch, fills the plain C argument struct (raw device pointers, strides, sizes) and calls
// the entry point on torch's current HIP stream.  Nothing is computed here.  The library itself is opened at
// run time (load_library), so the same extension serves libtah_duo.so and, in the CPU tests, the host build
// of the kernels.  There is no fallback: without a loaded library every call throws.
#include <c10/hip/HIPStream.h>
#include <dlfcn.h>
#include <torch/extension.h>

#include <string>
#include <tuple>

#include "tah_duo.h"

namespace {

using at::Tensor;
using c10::optional;

struct Api {
    void* handle = nullptr;
    bool allow_host = false;
    decltype(&tah_duo_abi_version) abi_version = nullptr;
    decltype(&tah_duo_error_string) error_string = nullptr;
    decltype(&tah_duo_fwd_varlen) fwd_varlen = nullptr;
    decltype(&tah_duo_bwd_varlen) bwd_varlen = nullptr;
    decltype(&tah_duo_bwd_workspace_bytes) bwd_workspace_bytes = nullptr;
    decltype(&tah_duo_schedule_bytes) schedule_bytes = nullptr;
    decltype(&tah_duo_schedule_build) schedule_build = nullptr;
    decltype(&tah_greedy_step) greedy_step = nullptr;
    decltype(&tah_silu_mul_normed) silu_mul_normed = nullptr;
    decltype(&tah_step_begin) step_begin = nullptr;
    decltype(&tah_greedy_tick) greedy_tick = nullptr;
    decltype(&tah_decider_tail) decider_tail = nullptr;
    decltype(&tah_linear_pack_weight) linear_pack_weight = nullptr;
    decltype(&tah_linear_pack_rows) linear_pack_rows = nullptr;
    decltype(&tah_linear_rows) linear_rows = nullptr;
    decltype(&tah_duo_fwd_masked) fwd_masked = nullptr;
    decltype(&tah_duo_bwd_masked) bwd_masked = nullptr;
    decltype(&tah_duo_decode_workspace_bytes) decode_workspace_bytes = nullptr;
    decltype(&tah_duo_decode) decode = nullptr;
    decltype(&tah_duo_decode_static) decode_static = nullptr;
    decltype(&tah_kv_append) kv_append = nullptr;
    decltype(&tah_qk_prep) qk_prep = nullptr;
    decltype(&tah_duo_decode_step) decode_step = nullptr;
    decltype(&tah_duo_decode_step_supported) decode_step_supported = nullptr;
    decltype(&tah_topk_mix) topk_mix = nullptr;
    decltype(&tah_qk_prep_bwd) qk_prep_bwd = nullptr;
    decltype(&tah_sample_rows) sample_rows = nullptr;
    decltype(&tah_silu_mul) silu_mul = nullptr;
    decltype(&tah_hard_index_build) hard_index_build = nullptr;
    decltype(&tah_pad_rows_build) pad_rows_build = nullptr;
    decltype(&tah_rows_copy) rows_copy = nullptr;
} g;

template <class F>
void bind(F& f, const char* name) {
    f = reinterpret_cast<F>(dlsym(g.handle, name));
    TORCH_CHECK(f != nullptr, "tah_amd: ", name, " is not exported by the loaded library");
}

void load_library(const std::string& path, bool allow_host) {
    void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
    TORCH_CHECK(h != nullptr, "tah_amd: cannot load ", path, ": ", dlerror(),
                " (the HIP library is not built? there is no CPU or PyTorch fallback)");
    g = Api{};
    g.handle = h;
    g.allow_host = allow_host;
    bind(g.abi_version, "tah_duo_abi_version");
    bind(g.error_string, "tah_duo_error_string");
    bind(g.fwd_varlen, "tah_duo_fwd_varlen");
    bind(g.bwd_varlen, "tah_duo_bwd_varlen");
    bind(g.bwd_workspace_bytes, "tah_duo_bwd_workspace_bytes");
    bind(g.schedule_bytes, "tah_duo_schedule_bytes");
    bind(g.schedule_build, "tah_duo_schedule_build");
    bind(g.greedy_step, "tah_greedy_step");
    bind(g.silu_mul_normed, "tah_silu_mul_normed");
    bind(g.step_begin, "tah_step_begin");
    bind(g.greedy_tick, "tah_greedy_tick");
    bind(g.decider_tail, "tah_decider_tail");
    bind(g.linear_pack_weight, "tah_linear_pack_weight");
    bind(g.linear_pack_rows, "tah_linear_pack_rows");
    bind(g.linear_rows, "tah_linear_rows");
    bind(g.fwd_masked, "tah_duo_fwd_masked");
    bind(g.bwd_masked, "tah_duo_bwd_masked");
    bind(g.decode_workspace_bytes, "tah_duo_decode_workspace_bytes");
    bind(g.decode, "tah_duo_decode");
    bind(g.decode_static, "tah_duo_decode_static");
    bind(g.kv_append, "tah_kv_append");
    bind(g.qk_prep, "tah_qk_prep");
    bind(g.decode_step, "tah_duo_decode_step");
    bind(g.decode_step_supported, "tah_duo_decode_step_supported");
    bind(g.topk_mix, "tah_topk_mix");
    bind(g.sample_rows, "tah_sample_rows");
    bind(g.qk_prep_bwd, "tah_qk_prep_bwd");
    bind(g.silu_mul, "tah_silu_mul");
    bind(g.hard_index_build, "tah_hard_index_build");
    bind(g.pad_rows_build, "tah_pad_rows_build");
    bind(g.rows_copy, "tah_rows_copy");
    const int got = g.abi_version();
    TORCH_CHECK(got == TAH_DUO_ABI_VERSION, "tah_amd: library ABI version ", got, ", extension built for ", TAH_DUO_ABI_VERSION);
}

void need_lib() { TORCH_CHECK(g.handle != nullptr, "tah_amd: no library loaded (tah_amd._lib.lib() loads libtah_duo.so)"); }

void check_rc(int rc, const char* what) {
    TORCH_CHECK(rc == 0, what, ": ", g.error_string(rc), " (code ", rc, ")");
}

// One device for all tensors; host tensors only when the loaded library is the host build of the kernels.
struct Dev {
    bool set = false;
    c10::Device dev{c10::kCPU};
    void see(const Tensor& t) {
        if (!t.defined()) return;
        TORCH_CHECK(t.is_cuda() || g.allow_host, "tah_amd ops need CUDA/HIP tensors (no CPU path exists)");
        if (!set) { dev = t.device(); set = true; }
        else TORCH_CHECK(t.device() == dev, "tensors on different devices: ", dev, " vs ", t.device());
    }
    void see(const optional<Tensor>& t) { if (t.has_value()) see(*t); }
    tah_stream_t stream() const {
        if (set && dev.is_cuda()) return static_cast<tah_stream_t>(c10::hip::getCurrentHIPStream(dev.index()).stream());
        return nullptr;
    }
};

const void* ptr(const Tensor& t) { return (!t.defined() || t.numel() == 0) ? nullptr : t.data_ptr(); }
void* mptr(const Tensor& t) { return (!t.defined() || t.numel() == 0) ? nullptr : t.data_ptr(); }
const void* ptr(const optional<Tensor>& t) { return t.has_value() ? ptr(*t) : nullptr; }

void thd(const Tensor& t, const char* name) {
    TORCH_CHECK(t.dim() == 3 && t.scalar_type() == at::kBFloat16, name, " must be a bf16 [rows, heads, head_dim] tensor");
    TORCH_CHECK(t.numel() == 0 || t.stride(2) == 1, name, ": head_dim must be contiguous");
}
void i32(const Tensor& t, const char* name) {
    TORCH_CHECK(t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 tensor");
}

void fill_stream(tah_duo_stream& s, const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& o, const Tensor& lse,
                 const Tensor& cu_q, const Tensor& cu_k, const Tensor* pos_q, const Tensor* pos_k) {
    s.q = ptr(q); s.k = ptr(k); s.v = ptr(v); s.o = mptr(o); s.lse = static_cast<float*>(mptr(lse));
    s.cu_q = static_cast<const int32_t*>(cu_q.data_ptr());
    s.cu_k = static_cast<const int32_t*>(cu_k.data_ptr());
    s.pos_q = pos_q ? static_cast<const int32_t*>(ptr(*pos_q)) : nullptr;
    s.pos_k = pos_k ? static_cast<const int32_t*>(ptr(*pos_k)) : nullptr;
    s.q_row_stride = q.stride(0); s.q_head_stride = q.stride(1);
    s.k_row_stride = k.stride(0); s.k_head_stride = k.stride(1);
    s.v_row_stride = v.stride(0); s.v_head_stride = v.stride(1);
    s.o_row_stride = o.stride(0); s.o_head_stride = o.stride(1);
    s.total_q = (int32_t)q.size(0); s.total_k = (int32_t)k.size(0);
}

const void* schedule_ptr(const optional<Tensor>& schedule) {
    if (!schedule.has_value()) return nullptr;
    TORCH_CHECK(schedule->scalar_type() == at::kInt && schedule->is_contiguous(), "schedule must be the int32 tensor duo_schedule returned");
    return ptr(*schedule);
}

// Launch-order table for the varlen calls that use these boundaries (tah_duo_schedule_build).
Tensor duo_schedule(const Tensor& cu_q1, const Tensor& cu_k1, const Tensor& cu_q2, const Tensor& cu_k2, const Tensor& pos_q2,
                    int64_t hq, int64_t hkv, int64_t total_q1, int64_t total_k1, int64_t total_k2) {
    need_lib();
    i32(cu_q1, "cu_q1"); i32(cu_k1, "cu_k1"); i32(cu_q2, "cu_q2"); i32(cu_k2, "cu_k2"); i32(pos_q2, "pos_q2");
    Dev d;
    for (const Tensor* t : {&cu_q1, &cu_k1, &cu_q2, &cu_k2, &pos_q2}) d.see(*t);
    const int64_t nseq = cu_q1.numel() - 1;
    TORCH_CHECK(cu_k1.numel() == nseq + 1 && cu_q2.numel() == nseq + 1 && cu_k2.numel() == nseq + 1,
                "cu_seqlens tensors must all have nseq+1 entries");
    tah_duo_schedule_args a{};
    a.cu_q1 = static_cast<const int32_t*>(cu_q1.data_ptr()); a.cu_k1 = static_cast<const int32_t*>(cu_k1.data_ptr());
    a.cu_q2 = static_cast<const int32_t*>(cu_q2.data_ptr()); a.cu_k2 = static_cast<const int32_t*>(cu_k2.data_ptr());
    a.pos_q2 = static_cast<const int32_t*>(ptr(pos_q2));
    a.nseq = (int32_t)nseq; a.hq = (int32_t)hq; a.hkv = (int32_t)hkv;
    a.total_q1 = (int32_t)total_q1; a.total_k1 = (int32_t)total_k1; a.total_q2 = (int32_t)pos_q2.numel(); a.total_k2 = (int32_t)total_k2;
    const size_t bytes = g.schedule_bytes(a.nseq, a.hq, a.hkv, a.total_q1, a.total_k1, a.total_q2, a.total_k2);
    TORCH_CHECK(bytes > 0, "duo_schedule: unsupported sizes");
    auto out = at::empty({(int64_t)(bytes / sizeof(int32_t))}, cu_q1.options());
    a.schedule = out.data_ptr(); a.schedule_bytes = bytes;
    check_rc(g.schedule_build(&a, d.stream()), "tah_duo_schedule_build");
    return out;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> duo_fwd_varlen(const Tensor& q1, const Tensor& k1, const Tensor& v1, const Tensor& cu_q1,
                                                          const Tensor& cu_k1, const Tensor& q2, const Tensor& k2, const Tensor& v2,
                                                          const Tensor& pos_q2, const Tensor& pos_k2, const Tensor& cu_q2,
                                                          const Tensor& cu_k2, double scale, const optional<Tensor>& schedule) {
    need_lib();
    thd(q1, "q1"); thd(k1, "k1"); thd(v1, "v1"); thd(q2, "q2"); thd(k2, "k2"); thd(v2, "v2");
    i32(cu_q1, "cu_q1"); i32(cu_k1, "cu_k1"); i32(cu_q2, "cu_q2"); i32(cu_k2, "cu_k2"); i32(pos_q2, "pos_q2"); i32(pos_k2, "pos_k2");
    Dev d;
    for (const Tensor* t : {&q1, &k1, &v1, &q2, &k2, &v2, &cu_q1, &cu_k1, &cu_q2, &cu_k2, &pos_q2, &pos_k2}) d.see(*t);
    d.see(schedule);
    const int64_t nseq = cu_q1.numel() - 1;
    TORCH_CHECK(cu_k1.numel() == nseq + 1 && cu_q2.numel() == nseq + 1 && cu_k2.numel() == nseq + 1,
                "cu_seqlens tensors must all have nseq+1 entries");
    TORCH_CHECK(pos_q2.numel() == q2.size(0) && pos_k2.numel() == k2.size(0) && k1.sizes() == v1.sizes() && k2.sizes() == v2.sizes(),
                "inconsistent row counts");
    const int64_t hq = q1.size(1), dd = q1.size(2);
    auto o1 = at::empty({q1.size(0), hq, dd}, q1.options());
    auto o2 = at::empty({q2.size(0), hq, dd}, q1.options());
    auto lse1 = at::empty({hq, q1.size(0)}, q1.options().dtype(at::kFloat));
    auto lse2 = at::empty({hq, q2.size(0)}, q1.options().dtype(at::kFloat));
    tah_duo_fwd_args a{};
    fill_stream(a.s1, q1, k1, v1, o1, lse1, cu_q1, cu_k1, nullptr, nullptr);
    fill_stream(a.s2, q2, k2, v2, o2, lse2, cu_q2, cu_k2, &pos_q2, &pos_k2);
    a.nseq = (int32_t)nseq; a.hq = (int32_t)hq; a.hkv = (int32_t)k1.size(1); a.d = (int32_t)dd; a.scale = (float)scale;
    a.schedule = schedule_ptr(schedule);
    check_rc(g.fwd_varlen(&a, d.stream()), "tah_duo_fwd_varlen");
    return {o1, lse1, o2, lse2};
}

void fill_bwd_stream(tah_duo_bwd_stream& s, const Tensor& d_o, const Tensor& dq, const Tensor& dk, const Tensor& dv, const Tensor& delta) {
    s.d_o = ptr(d_o); s.dq = mptr(dq); s.dk = mptr(dk); s.dv = mptr(dv); s.delta = static_cast<float*>(mptr(delta));
    s.do_row_stride = d_o.stride(0); s.do_head_stride = d_o.stride(1);
    s.dq_row_stride = dq.stride(0); s.dq_head_stride = dq.stride(1);
    s.dk_row_stride = dk.stride(0); s.dk_head_stride = dk.stride(1);
    s.dv_row_stride = dv.stride(0); s.dv_head_stride = dv.stride(1);
}

std::vector<Tensor> duo_bwd_varlen(const Tensor& q1, const Tensor& k1, const Tensor& v1, const Tensor& o1, const Tensor& lse1,
                                   const Tensor& do1, const Tensor& cu_q1, const Tensor& cu_k1, const Tensor& q2, const Tensor& k2,
                                   const Tensor& v2, const Tensor& o2, const Tensor& lse2, const Tensor& do2, const Tensor& pos_q2,
                                   const Tensor& pos_k2, const Tensor& cu_q2, const Tensor& cu_k2, double scale,
                                   const optional<Tensor>& schedule, const optional<Tensor>& ds_workspace,
                                   int64_t max_seqlen_k1, int64_t max_seqlen_k2) {
    need_lib();
    for (auto p : {std::make_pair(&q1, "q1"), {&k1, "k1"}, {&v1, "v1"}, {&o1, "o1"}, {&do1, "do1"}, {&q2, "q2"}, {&k2, "k2"},
                   {&v2, "v2"}, {&o2, "o2"}, {&do2, "do2"}})
        thd(*p.first, p.second);
    i32(cu_q1, "cu_q1"); i32(cu_k1, "cu_k1"); i32(cu_q2, "cu_q2"); i32(cu_k2, "cu_k2"); i32(pos_q2, "pos_q2"); i32(pos_k2, "pos_k2");
    Dev d;
    for (const Tensor* t : {&q1, &k1, &v1, &o1, &lse1, &do1, &q2, &k2, &v2, &o2, &lse2, &do2, &cu_q1, &cu_k1, &cu_q2, &cu_k2, &pos_q2, &pos_k2})
        d.see(*t);
    d.see(schedule);
    TORCH_CHECK(do1.sizes() == q1.sizes() && do2.sizes() == q2.sizes() && o1.sizes() == q1.sizes() && o2.sizes() == q2.sizes(),
                "o / dO shapes must match q");
    TORCH_CHECK(lse1.scalar_type() == at::kFloat && lse2.scalar_type() == at::kFloat && lse1.is_contiguous() && lse2.is_contiguous(),
                "lse must be contiguous float32 [Hq, rows]");
    const int64_t hq = q1.size(1);
    auto dq1 = at::empty(q1.sizes(), q1.options()), dk1 = at::empty(k1.sizes(), k1.options()), dv1 = at::empty(v1.sizes(), v1.options());
    auto dq2 = at::empty(q2.sizes(), q2.options()), dk2 = at::empty(k2.sizes(), k2.options()), dv2 = at::empty(v2.sizes(), v2.options());
    auto delta1 = at::empty({2, hq, q1.size(0)}, q1.options().dtype(at::kFloat));
    auto delta2 = at::empty({2, hq, q2.size(0)}, q1.options().dtype(at::kFloat));
    tah_duo_bwd_args a{};
    fill_stream(a.fwd.s1, q1, k1, v1, o1, lse1, cu_q1, cu_k1, nullptr, nullptr);
    fill_stream(a.fwd.s2, q2, k2, v2, o2, lse2, cu_q2, cu_k2, &pos_q2, &pos_k2);
    a.fwd.nseq = (int32_t)(cu_q1.numel() - 1); a.fwd.hq = (int32_t)hq; a.fwd.hkv = (int32_t)k1.size(1); a.fwd.d = (int32_t)q1.size(2);
    a.fwd.scale = (float)scale;
    a.fwd.schedule = schedule_ptr(schedule);
    fill_bwd_stream(a.g1, do1, dq1, dk1, dv1, delta1);
    fill_bwd_stream(a.g2, do2, dq2, dk2, dv2, delta2);
    if (ds_workspace && ds_workspace->defined() && ds_workspace->numel() > 0) {
        d.see(*ds_workspace);
        TORCH_CHECK(ds_workspace->is_contiguous(), "ds_workspace must be contiguous");
        a.ds_workspace = ds_workspace->data_ptr();
        a.ds_workspace_bytes = (size_t)ds_workspace->numel() * ds_workspace->element_size();
        a.max_seqlen_k1 = (int32_t)max_seqlen_k1;
        a.max_seqlen_k2 = (int32_t)max_seqlen_k2;
    }
    check_rc(g.bwd_varlen(&a, d.stream()), "tah_duo_bwd_varlen");
    return {dq1, dk1, dv1, dq2, dk2, dv2};
}

void fill_mask(tah_additive_mask& m, const Tensor& mask, int64_t nseq, int64_t hq, int64_t tq, int64_t tk) {
    TORCH_CHECK(mask.dim() == 4 && (mask.scalar_type() == at::kBFloat16 || mask.scalar_type() == at::kFloat),
                "additive mask must be a 4-D bf16 or float32 tensor (B|1, Hq|1, Tq, Tkv)");
    TORCH_CHECK((mask.size(0) == 1 || mask.size(0) == nseq) && (mask.size(1) == 1 || mask.size(1) == hq) && mask.size(2) == tq &&
                    mask.size(3) == tk,
                "additive mask shape ", mask.sizes(), " does not match (B=", nseq, ", Hq=", hq, ", Tq=", tq, ", Tkv=", tk, ")");
    m.mask = mask.data_ptr();
    m.seq_stride = mask.size(0) != 1 ? mask.stride(0) : 0;
    m.head_stride = mask.size(1) != 1 ? mask.stride(1) : 0;
    m.q_stride = mask.stride(2); m.k_stride = mask.stride(3);
    m.dtype = mask.scalar_type() == at::kFloat ? 1 : 0;
}

Tensor dense_cu(const Tensor& like, int64_t nseq, int64_t t) {
    return at::arange(0, (nseq + 1) * t, t, like.options().dtype(at::kInt));
}

std::tuple<Tensor, Tensor> duo_fwd_masked(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& mask, int64_t nseq, double scale) {
    need_lib();
    thd(q, "q"); thd(k, "k"); thd(v, "v");
    Dev d; d.see(q); d.see(k); d.see(v); d.see(mask);
    TORCH_CHECK(nseq > 0 && q.size(0) % nseq == 0 && k.size(0) % nseq == 0 && k.sizes() == v.sizes(),
                "row counts must be multiples of the batch size");
    const int64_t tq = q.size(0) / nseq, tk = k.size(0) / nseq, hq = q.size(1), dd = q.size(2);
    auto o = at::empty({q.size(0), hq, dd}, q.options());
    auto lse = at::empty({hq, q.size(0)}, q.options().dtype(at::kFloat));
    auto cu_q = dense_cu(q, nseq, tq), cu_k = dense_cu(q, nseq, tk);
    auto zc = at::zeros({nseq + 1}, q.options().dtype(at::kInt));
    auto e = q.narrow(0, 0, 0), ek = k.narrow(0, 0, 0), el = lse.narrow(1, 0, 0);
    tah_duo_fwd_args a{};
    fill_stream(a.s1, q, k, v, o, lse, cu_q, cu_k, nullptr, nullptr);
    fill_stream(a.s2, e, ek, ek, e, el, zc, zc, nullptr, nullptr);
    a.nseq = (int32_t)nseq; a.hq = (int32_t)hq; a.hkv = (int32_t)k.size(1); a.d = (int32_t)dd; a.scale = (float)scale;
    tah_additive_mask m{};
    fill_mask(m, mask, nseq, hq, tq, tk);
    check_rc(g.fwd_masked(&a, &m, d.stream()), "tah_duo_fwd_masked");
    return {o, lse};
}

std::vector<Tensor> duo_bwd_masked(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& o, const Tensor& lse,
                                   const Tensor& d_o, const Tensor& mask, int64_t nseq, double scale) {
    need_lib();
    thd(q, "q"); thd(k, "k"); thd(v, "v"); thd(o, "o"); thd(d_o, "d_o");
    Dev d;
    for (const Tensor* t : {&q, &k, &v, &o, &lse, &d_o, &mask}) d.see(*t);
    TORCH_CHECK(d_o.sizes() == q.sizes() && o.sizes() == q.sizes(), "o / dO shapes must match q");
    TORCH_CHECK(lse.scalar_type() == at::kFloat && lse.is_contiguous(), "lse must be contiguous float32 [Hq, rows]");
    const int64_t tq = q.size(0) / nseq, tk = k.size(0) / nseq, hq = q.size(1);
    auto dq = at::empty(q.sizes(), q.options()), dk = at::empty(k.sizes(), k.options()), dv = at::empty(v.sizes(), v.options());
    auto delta = at::empty({2, hq, q.size(0)}, q.options().dtype(at::kFloat));
    auto cu_q = dense_cu(q, nseq, tq), cu_k = dense_cu(q, nseq, tk);
    auto zc = at::zeros({nseq + 1}, q.options().dtype(at::kInt));
    auto e = q.narrow(0, 0, 0), ek = k.narrow(0, 0, 0), el = lse.narrow(1, 0, 0), ed = delta.narrow(2, 0, 0);
    tah_duo_bwd_args a{};
    fill_stream(a.fwd.s1, q, k, v, o, lse, cu_q, cu_k, nullptr, nullptr);
    fill_stream(a.fwd.s2, e, ek, ek, e, el, zc, zc, nullptr, nullptr);
    a.fwd.nseq = (int32_t)nseq; a.fwd.hq = (int32_t)hq; a.fwd.hkv = (int32_t)k.size(1); a.fwd.d = (int32_t)q.size(2); a.fwd.scale = (float)scale;
    fill_bwd_stream(a.g1, d_o, dq, dk, dv, delta);
    fill_bwd_stream(a.g2, e, e, ek, ek, ed);
    tah_additive_mask m{};
    fill_mask(m, mask, nseq, hq, tq, tk);
    check_rc(g.bwd_masked(&a, &m, d.stream()), "tah_duo_bwd_masked");
    return {dq, dk, dv};
}

// One depth of the slab cache as tensors: k, v [slot, Hkv, capacity, D]; pos [slot, capacity] or none; start, len [slot].
tah_kv_segment segment(const Tensor& k, const Tensor& v, const optional<Tensor>& pos, const Tensor& start, const Tensor& len) {
    TORCH_CHECK(k.dim() == 4 && v.sizes() == k.sizes() && k.is_contiguous() && v.is_contiguous(), "slabs must be contiguous [slot, Hkv, capacity, D]");
    tah_kv_segment s{};
    s.k = k.data_ptr(); s.v = v.data_ptr();
    s.pos = pos.has_value() ? static_cast<int32_t*>(pos->data_ptr()) : nullptr;
    s.start = static_cast<const int32_t*>(start.data_ptr());
    s.len = static_cast<int32_t*>(len.data_ptr());
    s.k_row_stride = s.v_row_stride = k.size(3);
    s.k_head_stride = s.v_head_stride = k.size(2) * k.size(3);
    s.capacity = (int32_t)k.size(2);
    s.nslots = (int32_t)k.size(0);
    return s;
}

int64_t decode_workspace_bytes(int64_t nq, int64_t hq, int64_t cap1, int64_t cap2) {
    need_lib();
    return (int64_t)g.decode_workspace_bytes((int32_t)nq, (int32_t)hq, (int32_t)cap1, (int32_t)cap2);
}

// tah_duo_decode_args from tensors; q may be absent for the fused step (the queries are prepared inside the kernel).
tah_duo_decode_args decode_args(Dev& d, const optional<Tensor>& q, const Tensor& o, const optional<Tensor>& lse, const Tensor& q_slot,
                                const Tensor& q_pos, const optional<Tensor>& q_depth, int64_t depth, const Tensor& k1, const Tensor& v1,
                                const Tensor& start1, const Tensor& len1, const optional<Tensor>& k2, const optional<Tensor>& v2,
                                const optional<Tensor>& pos2, const optional<Tensor>& start2, const optional<Tensor>& len2, double scale,
                                const optional<Tensor>& o_packed) {
    thd(o, "o"); i32(q_slot, "q_slot"); i32(q_pos, "q_pos");
    d.see(q); d.see(o); d.see(lse); d.see(q_slot); d.see(q_pos); d.see(q_depth); d.see(k1); d.see(o_packed);
    if (o_packed.has_value())
        TORCH_CHECK(o_packed->scalar_type() == at::kBFloat16 && o_packed->is_contiguous() && o_packed->numel() == 32 * o.size(1) * o.size(2),
                    "duo_decode: o_packed must be a contiguous bf16 tensor of 32 * Hq * D elements");
    const bool need2 = q_depth.has_value() || depth >= 1;
    TORCH_CHECK(!need2 || (k2.has_value() && v2.has_value() && pos2.has_value() && start2.has_value() && len2.has_value()),
                "depth-1 queries need the depth-1 cache");
    tah_duo_decode_args a{};
    a.o = mptr(o); a.lse = lse.has_value() ? static_cast<float*>(lse->data_ptr()) : nullptr;
    a.o_row_stride = o.stride(0); a.o_head_stride = o.stride(1);
    if (q.has_value()) {
        thd(*q, "q");
        TORCH_CHECK(q->sizes() == o.sizes(), "duo_decode: q and o must have the same shape");
        a.q = ptr(*q); a.q_row_stride = q->stride(0); a.q_head_stride = q->stride(1);
    }
    a.q_slot = static_cast<const int32_t*>(q_slot.data_ptr());
    a.q_pos = static_cast<const int32_t*>(q_pos.data_ptr());
    a.q_depth = q_depth.has_value() ? static_cast<const int32_t*>(q_depth->data_ptr()) : nullptr;
    a.depth = (int32_t)depth;
    a.c1 = segment(k1, v1, c10::nullopt, start1, len1);
    if (need2) a.c2 = segment(*k2, *v2, pos2, *start2, *len2);
    a.nq = (int32_t)o.size(0); a.hq = (int32_t)o.size(1); a.hkv = (int32_t)k1.size(1); a.d = (int32_t)o.size(2); a.scale = (float)scale;
    a.o_packed = o_packed.has_value() ? o_packed->data_ptr() : nullptr;
    return a;
}

void duo_decode(const Tensor& q, const Tensor& o, const optional<Tensor>& lse, const Tensor& q_slot, const Tensor& q_pos,
                const optional<Tensor>& q_depth, int64_t depth, const Tensor& k1, const Tensor& v1, const Tensor& start1,
                const Tensor& len1, const optional<Tensor>& k2, const optional<Tensor>& v2, const optional<Tensor>& pos2,
                const optional<Tensor>& start2, const optional<Tensor>& len2, const optional<Tensor>& workspace, double scale,
                const optional<Tensor>& o_packed) {
    need_lib();
    Dev d; d.see(workspace);
    tah_duo_decode_args a = decode_args(d, q, o, lse, q_slot, q_pos, q_depth, depth, k1, v1, start1, len1, k2, v2, pos2, start2, len2, scale, o_packed);
    if (workspace.has_value()) {
        a.workspace = workspace->data_ptr();
        a.workspace_bytes = (size_t)workspace->numel() * workspace->element_size();
        check_rc(g.decode(&a, d.stream()), "tah_duo_decode");
    } else {
        check_rc(g.decode_static(&a, d.stream()), "tah_duo_decode_static");
    }
}

void kv_append(const Tensor& k_new, const Tensor& v_new, const Tensor& cu_new, const optional<Tensor>& pos_new,
               const optional<Tensor>& slot_of, const Tensor& ck, const Tensor& cv, const optional<Tensor>& cpos, const Tensor& start,
               const Tensor& len, const Tensor& overflow) {
    need_lib();
    thd(k_new, "k_new"); thd(v_new, "v_new"); i32(cu_new, "cu_new");
    Dev d; d.see(k_new); d.see(v_new); d.see(cu_new); d.see(pos_new); d.see(slot_of); d.see(ck);
    TORCH_CHECK(pos_new.has_value() == cpos.has_value(), "pos_new must be given exactly for slabs created with_pos=True");
    tah_kv_append_args a{};
    a.k_new = ptr(k_new); a.v_new = ptr(v_new); a.pos_new = static_cast<const int32_t*>(ptr(pos_new));
    a.k_row_stride = k_new.stride(0); a.k_head_stride = k_new.stride(1);
    a.v_row_stride = v_new.stride(0); a.v_head_stride = v_new.stride(1);
    a.cu_new = static_cast<const int32_t*>(cu_new.data_ptr());
    a.slot_of = static_cast<const int32_t*>(ptr(slot_of));
    a.nseq = (int32_t)(cu_new.numel() - 1); a.total_new = (int32_t)k_new.size(0); a.hkv = (int32_t)ck.size(1); a.d = (int32_t)ck.size(3);
    a.cache = segment(ck, cv, cpos, start, len);
    a.overflow = static_cast<int32_t*>(overflow.data_ptr());
    check_rc(g.kv_append(&a, d.stream()), "tah_kv_append");
}

// tah_qk_prep_args from tensors; q_out may be absent for the fused step (the prepared heads stay in registers).
tah_qk_prep_args prep_args(Dev& d, const Tensor& q, const Tensor& k, const optional<Tensor>& v, const optional<Tensor>& q_out,
                           const optional<Tensor>& k_out, const Tensor& q_weight, const Tensor& k_weight, const Tensor& cos,
                           const Tensor& sin, double eps, const optional<Tensor>& ck, const optional<Tensor>& cv,
                           const optional<Tensor>& cpos, const optional<Tensor>& start, const optional<Tensor>& len,
                           const optional<Tensor>& overflow, const optional<Tensor>& cu_new, const optional<Tensor>& pos_new,
                           const optional<Tensor>& slot_of, bool one_row_per_seq, const optional<Tensor>& v_out,
                           const optional<Tensor>& norm_input, double norm_eps) {
    thd(q, "q"); thd(k, "k");
    d.see(q); d.see(k); d.see(v); d.see(q_weight); d.see(k_weight); d.see(cos); d.see(sin); d.see(cu_new); d.see(pos_new);
    d.see(slot_of); d.see(ck);
    const int64_t D = q.size(2);
    for (auto p : {std::make_pair(&q_weight, "q_weight"), {&k_weight, "k_weight"}})
        TORCH_CHECK(p.first->scalar_type() == at::kBFloat16 && p.first->dim() == 1 && p.first->size(0) == D && p.first->is_contiguous(),
                    p.second, " must be a contiguous bf16 [", D, "] tensor");
    for (auto p : {std::make_pair(&cos, "cos"), {&sin, "sin"}})
        TORCH_CHECK(p.first->scalar_type() == at::kBFloat16 && p.first->dim() == 2 && p.first->size(0) == q.size(0) &&
                        p.first->size(1) == D && p.first->stride(1) == 1,
                    p.second, " must be a bf16 [rows, ", D, "] tensor with unit inner stride");
    TORCH_CHECK(cos.stride(0) == sin.stride(0), "cos and sin must share their row stride");
    TORCH_CHECK(k.size(0) == q.size(0), "q and k must have one row per token");
    tah_qk_prep_args a{};
    a.q = ptr(q); a.k = ptr(k); a.v = ptr(v);
    a.q_row_stride = q.stride(0); a.q_head_stride = q.stride(1);
    a.k_row_stride = k.stride(0); a.k_head_stride = k.stride(1);
    if (q_out.has_value()) {
        thd(*q_out, "q_out");
        a.q_out = mptr(*q_out);
        a.q_out_row_stride = q_out->stride(0); a.q_out_head_stride = q_out->stride(1);
    }
    if (v.has_value()) { thd(*v, "v"); a.v_row_stride = v->stride(0); a.v_head_stride = v->stride(1); }
    a.q_weight = ptr(q_weight); a.k_weight = ptr(k_weight); a.cos = ptr(cos); a.sin = ptr(sin);
    a.cos_sin_row_stride = cos.stride(0);
    a.eps = (float)eps;
    a.rows = (int32_t)q.size(0); a.hq = (int32_t)q.size(1); a.hkv = (int32_t)k.size(1); a.d = (int32_t)D;
    if (ck.has_value()) {
        TORCH_CHECK(v.has_value() && cu_new.has_value(), "appending needs v and cu_new");
        TORCH_CHECK(pos_new.has_value() == cpos.has_value(), "pos_new must be given exactly for slabs created with_pos=True");
        i32(*cu_new, "cu_new");
        a.append = 1;
        a.append_one_row_per_seq = one_row_per_seq ? 1 : 0;
        a.cu_new = static_cast<const int32_t*>(cu_new->data_ptr());
        a.slot_of = static_cast<const int32_t*>(ptr(slot_of));
        a.pos_new = static_cast<const int32_t*>(ptr(pos_new));
        a.nseq = (int32_t)(cu_new->numel() - 1);
        a.cache = segment(*ck, *cv, cpos, *start, *len);
        a.overflow = overflow.has_value() ? static_cast<int32_t*>(overflow->data_ptr()) : nullptr;
    } else {
        TORCH_CHECK(k_out.has_value(), "k_out is needed when nothing is appended");
        a.k_out = mptr(*k_out);
        a.k_out_row_stride = k_out->stride(0); a.k_out_head_stride = k_out->stride(1);
        if (v_out.has_value()) {
            TORCH_CHECK(v.has_value() && v_out->sizes() == v->sizes(), "v_out needs v, and its shape");
            thd(*v_out, "v_out");
            d.see(v_out);
            a.v_out = mptr(*v_out);
            a.v_out_row_stride = v_out->stride(0); a.v_out_head_stride = v_out->stride(1);
        }
    }
    if (norm_input.has_value()) {
        d.see(norm_input);
        TORCH_CHECK(norm_input->dim() == 2 && norm_input->scalar_type() == at::kBFloat16 && norm_input->size(0) == q.size(0) &&
                        norm_input->stride(1) == 1,
                    "norm_input must be a bf16 [rows, hidden] tensor with unit inner stride");
        a.norm_input = ptr(*norm_input);
        a.norm_input_row_stride = norm_input->size(0) > 1 ? norm_input->stride(0) : norm_input->size(1);
        a.norm_cols = (int32_t)norm_input->size(1);
        a.norm_eps = (float)norm_eps;
    }
    return a;
}

// q/k RMSNorm + rotary (+ append): returns nothing, the caller allocated q_out / k_out.
void qk_prep(const Tensor& q, const Tensor& k, const optional<Tensor>& v, const Tensor& q_out, const optional<Tensor>& k_out,
             const Tensor& q_weight, const Tensor& k_weight, const Tensor& cos, const Tensor& sin, double eps,
             const optional<Tensor>& ck, const optional<Tensor>& cv, const optional<Tensor>& cpos, const optional<Tensor>& start,
             const optional<Tensor>& len, const optional<Tensor>& overflow, const optional<Tensor>& cu_new,
             const optional<Tensor>& pos_new, const optional<Tensor>& slot_of, bool one_row_per_seq,
             const optional<Tensor>& v_out, const optional<Tensor>& norm_input, double norm_eps) {
    need_lib();
    Dev d;
    const tah_qk_prep_args a = prep_args(d, q, k, v, q_out, k_out, q_weight, k_weight, cos, sin, eps, ck, cv, cpos, start, len, overflow,
                                         cu_new, pos_new, slot_of, one_row_per_seq, v_out, norm_input, norm_eps);
    check_rc(g.qk_prep(&a, d.stream()), "tah_qk_prep");
}

// backward of qk_prep (no append, no folded input norm): returns dq, dk (bf16) and the per-workgroup partial sums of the
// two weight gradients, float32 [n_partial, 2, D]
std::vector<Tensor> qk_prep_bwd(const Tensor& q, const Tensor& k, const Tensor& dq_out, const Tensor& dk_out, const Tensor& q_weight,
                                const Tensor& k_weight, const Tensor& cos, const Tensor& sin, double eps, int64_t n_partial) {
    need_lib();
    Dev d;
    thd(q, "q"); thd(k, "k"); thd(dq_out, "dq_out"); thd(dk_out, "dk_out");
    d.see(q); d.see(k); d.see(dq_out); d.see(dk_out); d.see(q_weight); d.see(k_weight); d.see(cos); d.see(sin);
    const int64_t D = q.size(2), rows = q.size(0);
    TORCH_CHECK(dq_out.sizes() == q.sizes() && dk_out.sizes() == k.sizes() && k.size(0) == rows, "qk_prep_bwd: gradient shapes must match q and k");
    for (auto p : {std::make_pair(&q_weight, "q_weight"), {&k_weight, "k_weight"}})
        TORCH_CHECK(p.first->scalar_type() == at::kBFloat16 && p.first->dim() == 1 && p.first->size(0) == D && p.first->is_contiguous(),
                    p.second, " must be a contiguous bf16 [", D, "] tensor");
    for (auto p : {std::make_pair(&cos, "cos"), {&sin, "sin"}})
        TORCH_CHECK(p.first->scalar_type() == at::kBFloat16 && p.first->dim() == 2 && p.first->size(0) == rows && p.first->size(1) == D &&
                        p.first->stride(1) == 1,
                    p.second, " must be a bf16 [rows, ", D, "] tensor with unit inner stride");
    TORCH_CHECK(cos.stride(0) == sin.stride(0), "cos and sin must share their row stride");
    TORCH_CHECK(n_partial >= 1, "qk_prep_bwd: n_partial must be at least 1");
    Tensor dq = at::empty(q.sizes(), q.options()), dk = at::empty(k.sizes(), k.options());
    Tensor part = at::empty({n_partial, 2, D}, q.options().dtype(at::kFloat));
    tah_qk_prep_bwd_args a{};
    a.q = ptr(q); a.k = ptr(k); a.dq_out = ptr(dq_out); a.dk_out = ptr(dk_out); a.dq = dq.data_ptr(); a.dk = dk.data_ptr();
    a.q_row_stride = q.stride(0); a.q_head_stride = q.stride(1); a.k_row_stride = k.stride(0); a.k_head_stride = k.stride(1);
    a.dq_out_row_stride = dq_out.stride(0); a.dq_out_head_stride = dq_out.stride(1);
    a.dk_out_row_stride = dk_out.stride(0); a.dk_out_head_stride = dk_out.stride(1);
    a.dq_row_stride = dq.stride(0); a.dq_head_stride = dq.stride(1); a.dk_row_stride = dk.stride(0); a.dk_head_stride = dk.stride(1);
    a.q_weight = ptr(q_weight); a.k_weight = ptr(k_weight); a.cos = ptr(cos); a.sin = ptr(sin);
    a.cos_sin_row_stride = cos.stride(0);
    a.eps = (float)eps;
    a.rows = (int32_t)rows; a.hq = (int32_t)q.size(1); a.hkv = (int32_t)k.size(1); a.d = (int32_t)D;
    a.dw_partial = static_cast<float*>(part.data_ptr());
    a.n_partial = (int32_t)n_partial;
    check_rc(g.qk_prep_bwd(&a, d.stream()), "tah_qk_prep_bwd");
    return {dq, dk, part};
}

bool duo_decode_step_supported(int64_t nq, int64_t hq, int64_t hkv, int64_t capacity1) {
    need_lib();
    return g.decode_step_supported((int32_t)nq, (int32_t)hq, (int32_t)hkv, (int32_t)capacity1) != 0;
}

// qk_prep (append, one row per sequence) + duo_decode in one launch (tah_duo_decode_step).  The slabs the new K/V go to
// (ck, cv, ...) must be those of one of the two segments read.
void duo_decode_step(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& q_weight, const Tensor& k_weight,
                     const Tensor& cos, const Tensor& sin, double eps, const Tensor& ck, const Tensor& cv,
                     const optional<Tensor>& cpos, const Tensor& start, const Tensor& len, const optional<Tensor>& overflow,
                     const Tensor& cu_new, const optional<Tensor>& pos_new, const optional<Tensor>& slot_of,
                     const optional<Tensor>& norm_input, double norm_eps, const Tensor& append_at,
                     const optional<Tensor>& append_depth, const Tensor& o, const optional<Tensor>& lse, const Tensor& q_slot, const Tensor& q_pos,
                     const optional<Tensor>& q_depth, int64_t depth, const Tensor& k1, const Tensor& v1, const Tensor& start1,
                     const Tensor& len1, const optional<Tensor>& k2, const optional<Tensor>& v2, const optional<Tensor>& pos2,
                     const optional<Tensor>& start2, const optional<Tensor>& len2, double scale, const optional<Tensor>& o_packed) {
    need_lib();
    Dev d; d.see(append_at); d.see(append_depth);
    i32(append_at, "append_at");
    TORCH_CHECK(append_at.numel() == q.size(0), "duo_decode_step: append_at must have one entry per row");
    if (append_depth.has_value()) {
        i32(*append_depth, "append_depth");
        TORCH_CHECK(append_depth->numel() == q.size(0), "duo_decode_step: append_depth must have one entry per row");
    }
    const tah_qk_prep_args pa = prep_args(d, q, k, v, c10::nullopt, c10::nullopt, q_weight, k_weight, cos, sin, eps, ck, cv, cpos, start, len,
                                          overflow, cu_new, pos_new, slot_of, true, c10::nullopt, norm_input, norm_eps);
    const tah_duo_decode_args da = decode_args(d, c10::nullopt, o, lse, q_slot, q_pos, q_depth, depth, k1, v1, start1, len1, k2, v2, pos2,
                                               start2, len2, scale, o_packed);
    check_rc(g.decode_step(&pa, &da, static_cast<const int32_t*>(append_at.data_ptr()),
                           append_depth.has_value() ? static_cast<const int32_t*>(append_depth->data_ptr()) : nullptr, d.stream()),
             "tah_duo_decode_step");
}

std::tuple<Tensor, Tensor, Tensor, Tensor> hard_index_build(const Tensor& mask) {
    need_lib();
    Dev d; d.see(mask);
    TORCH_CHECK(mask.dim() == 2 && (mask.scalar_type() == at::kBool || mask.scalar_type() == at::kByte),
                "mask must be a (B, S) bool or uint8 tensor");
    auto m = mask.contiguous();
    const int64_t B = m.size(0), S = m.size(1), cap = std::max<int64_t>(B * S, 1);
    auto io = m.options().dtype(at::kInt);
    auto pos = at::empty({cap}, io), flat = at::empty({cap}, io), seq = at::empty({cap}, io), cu = at::empty({B + 1}, io);
    check_rc(g.hard_index_build(static_cast<const uint8_t*>(ptr(m)), (int32_t)B, (int32_t)S, static_cast<int32_t*>(pos.data_ptr()),
                                static_cast<int32_t*>(flat.data_ptr()), static_cast<int32_t*>(seq.data_ptr()),
                                static_cast<int32_t*>(cu.data_ptr()), d.stream()),
             "tah_hard_index_build");
    return {pos, flat, seq, cu};
}

Tensor pad_rows_build(const Tensor& cu, const Tensor& seq_of, int64_t n, int64_t width, const optional<Tensor>& n_dev,
                      const optional<Tensor>& overflow) {
    need_lib();
    Dev d; d.see(cu); d.see(seq_of); d.see(n_dev); d.see(overflow);
    auto out = at::empty({std::max<int64_t>(n, 1)}, cu.options().dtype(at::kInt));
    check_rc(g.pad_rows_build(static_cast<const int32_t*>(cu.data_ptr()), static_cast<const int32_t*>(seq_of.data_ptr()), (int32_t)n,
                              static_cast<const int32_t*>(ptr(n_dev)), (int32_t)width, static_cast<int32_t*>(out.data_ptr()),
                              overflow.has_value() ? static_cast<int32_t*>(overflow->data_ptr()) : nullptr, d.stream()),
             "tah_pad_rows_build");
    return out.narrow(0, 0, n);
}

void rows_copy(const Tensor& src, const optional<Tensor>& src_rows, const Tensor& dst, const optional<Tensor>& dst_rows, int64_t n,
               const optional<Tensor>& dst_enable, const optional<Tensor>& n_dev) {
    need_lib();
    Dev d; d.see(src); d.see(dst); d.see(src_rows); d.see(dst_rows); d.see(dst_enable); d.see(n_dev);
    if (dst_enable.has_value())
        TORCH_CHECK((dst_enable->scalar_type() == at::kBool || dst_enable->scalar_type() == at::kByte) && dst_enable->is_contiguous() &&
                        dst_enable->numel() == dst.size(0),
                    "rows_copy: dst_enable must be a contiguous bool/uint8 tensor with one entry per dst row");
    if (n == 0) return;
    TORCH_CHECK(src.scalar_type() == dst.scalar_type() && src.sizes().slice(1) == dst.sizes().slice(1),
                "rows_copy: src and dst rows differ in dtype or shape");
    TORCH_CHECK(src.select(0, 0).is_contiguous() && dst.select(0, 0).is_contiguous(), "rows_copy: rows must be contiguous");
    const int64_t row_elems = src.select(0, 0).numel(), es = src.element_size();
    const int64_t sstride = (src.size(0) > 1 ? src.stride(0) : row_elems) * es;
    const int64_t dstride = (dst.size(0) > 1 ? dst.stride(0) : row_elems) * es;
    check_rc(g.rows_copy(src.data_ptr(), static_cast<const int32_t*>(ptr(src_rows)), dst.data_ptr(),
                         static_cast<const int32_t*>(ptr(dst_rows)), static_cast<const uint8_t*>(ptr(dst_enable)), (int32_t)n,
                         static_cast<const int32_t*>(ptr(n_dev)), row_elems * es, sstride, dstride, d.stream()),
             "tah_rows_copy");
}

Tensor topk_mix(const Tensor& logits, const Tensor& embedding, int64_t topk, const optional<Tensor>& row_enable, const optional<Tensor>& out_,
                const optional<Tensor>& out_packed, bool zero_disabled, const optional<Tensor>& values_out) {
    need_lib();
    Dev d; d.see(logits); d.see(embedding); d.see(row_enable); d.see(out_); d.see(out_packed); d.see(values_out);
    TORCH_CHECK(logits.dim() == 2 && embedding.dim() == 2 && logits.scalar_type() == at::kBFloat16 && embedding.scalar_type() == at::kBFloat16,
                "topk_mix: logits [rows, V] and embedding [V, H] must be bf16");
    TORCH_CHECK(logits.size(1) == embedding.size(0) && logits.stride(1) == 1 && embedding.stride(1) == 1,
                "topk_mix: vocabulary sizes differ or the inner dimension is not contiguous");
    const int64_t rows = logits.size(0), H = embedding.size(1);
    // rows that are not enabled: zeros in a fresh tensor (it is zero-filled); in the caller's tensor they keep their
    // contents unless zero_disabled asks the kernel to write zeros
    Tensor out = out_.has_value() ? *out_ : (row_enable.has_value() ? at::zeros({rows, H}, embedding.options()) : at::empty({rows, H}, embedding.options()));
    if (out_packed.has_value())
        TORCH_CHECK(out_packed->scalar_type() == at::kBFloat16 && out_packed->is_contiguous() && out_packed->numel() == 32 * H,
                    "topk_mix: out_packed must be a contiguous bf16 tensor of 32 * H elements");
    TORCH_CHECK(out.dim() == 2 && out.size(0) == rows && out.size(1) == H && out.scalar_type() == embedding.scalar_type() && out.stride(1) == 1,
                "topk_mix: out must be bf16 [rows, H]");
    if (row_enable.has_value())
        TORCH_CHECK((row_enable->scalar_type() == at::kBool || row_enable->scalar_type() == at::kByte) && row_enable->numel() == rows &&
                        row_enable->is_contiguous(),
                    "topk_mix: row_enable must be a contiguous bool/uint8 [rows] tensor");
    tah_topk_mix_args a{};
    a.logits = ptr(logits); a.embedding = ptr(embedding); a.out = mptr(out);
    a.row_enable = static_cast<const uint8_t*>(ptr(row_enable));
    a.logits_row_stride = rows > 1 ? logits.stride(0) : logits.size(1);
    a.embedding_row_stride = embedding.stride(0);
    a.out_row_stride = rows > 1 ? out.stride(0) : H;
    a.rows = (int32_t)rows; a.vocab = (int32_t)logits.size(1); a.hidden = (int32_t)H; a.topk = (int32_t)topk;
    a.out_packed = out_packed.has_value() ? out_packed->data_ptr() : nullptr;
    a.zero_disabled = zero_disabled ? 1 : 0;
    if (values_out.has_value()) {
        TORCH_CHECK(values_out->dim() == 2 && values_out->size(0) == rows && values_out->size(1) == std::min<int64_t>(topk, logits.size(1)) &&
                        values_out->scalar_type() == at::kBFloat16 && values_out->stride(1) == 1,
                    "topk_mix: values_out must be bf16 [rows, min(topk, V)]");
        a.values_out = values_out->data_ptr();
        a.values_row_stride = rows > 1 ? values_out->stride(0) : values_out->size(1);
    }
    check_rc(g.topk_mix(&a, d.stream()), "tah_topk_mix");
    return out;
}

// the top-k logits of every row, largest first (tah_topk_mix with values_out only), optionally with their indices
// (`out`: a bf16 [rows, >= k] matrix whose first k columns receive the values, e.g. rows padded for a linear layer)
Tensor topk_values(const Tensor& logits, int64_t topk, const optional<Tensor>& indices, const optional<Tensor>& out) {
    need_lib();
    Dev d; d.see(logits); d.see(out);
    TORCH_CHECK(logits.dim() == 2 && logits.scalar_type() == at::kBFloat16 && logits.stride(1) == 1 && topk >= 1,
                "topk_values: logits must be bf16 [rows, V] with a contiguous inner dimension");
    const int64_t rows = logits.size(0), k = std::min<int64_t>(topk, logits.size(1));
    if (out.has_value())
        TORCH_CHECK(out->dim() == 2 && out->scalar_type() == at::kBFloat16 && out->size(0) == rows && out->size(1) >= k &&
                        (out->numel() == 0 || out->stride(1) == 1),
                    "topk_values: out must be bf16 [rows, >= min(topk, V)] with a contiguous inner dimension");
    Tensor vals = out.has_value() ? *out : at::empty({rows, k}, logits.options());
    tah_topk_mix_args a{};
    a.logits = ptr(logits);
    a.logits_row_stride = rows > 1 ? logits.stride(0) : logits.size(1);
    a.rows = (int32_t)rows; a.vocab = (int32_t)logits.size(1); a.hidden = 8; a.topk = (int32_t)topk;
    a.values_out = vals.data_ptr();
    a.values_row_stride = out.has_value() && rows > 1 ? out->stride(0) : vals.size(1);
    if (indices.has_value()) {
        TORCH_CHECK(!out.has_value() || a.values_row_stride == k, "topk_values: indices go with values rows of exactly min(topk, V) columns");
        d.see(*indices);
        TORCH_CHECK(indices->scalar_type() == at::kInt && indices->dim() == 2 && indices->size(0) == rows && indices->size(1) == k && indices->is_contiguous(),
                    "topk_values: indices must be a contiguous int32 [rows, min(topk, V)] tensor");
        a.indices_out = static_cast<int32_t*>(indices->data_ptr());
    }
    check_rc(g.topk_mix(&a, d.stream()), "tah_topk_mix");
    return vals;
}

// one token per row by temperature / min_p / top_p sampling (tah_sample_rows); returns tokens int64 [rows], and fills
// `probs_out` (float32 [rows, V]) with the distribution drawn from when it is given; without `uniforms` only that
void sample_rows(const Tensor& logits, const optional<Tensor>& logits_prev, const optional<Tensor>& add_prev,
                 const optional<Tensor>& uniforms, const optional<Tensor>& tokens_out, const optional<Tensor>& probs_out,
                 const optional<Tensor>& row_enable, double temperature, double top_p, double min_p) {
    need_lib();
    Dev d; d.see(logits);
    TORCH_CHECK(logits.dim() == 2 && logits.scalar_type() == at::kBFloat16 && logits.stride(1) == 1,
                "sample_rows: logits must be bf16 [rows, V] with a contiguous inner dimension");
    const int64_t rows = logits.size(0), V = logits.size(1);
    tah_sample_rows_args a{};
    a.logits = ptr(logits);
    a.logits_row_stride = rows > 1 ? logits.stride(0) : V;
    if (logits_prev.has_value()) {
        d.see(*logits_prev);
        TORCH_CHECK(logits_prev->sizes() == logits.sizes() && logits_prev->scalar_type() == at::kBFloat16 && logits_prev->stride(1) == 1,
                    "sample_rows: logits_prev must be bf16 [rows, V] like logits");
        TORCH_CHECK(add_prev.has_value(), "sample_rows: logits_prev needs add_prev");
        a.logits_prev = ptr(*logits_prev);
        a.prev_row_stride = rows > 1 ? logits_prev->stride(0) : V;
    }
    if (add_prev.has_value()) {
        d.see(*add_prev);
        TORCH_CHECK(add_prev->scalar_type() == at::kInt && add_prev->is_contiguous() && add_prev->numel() == rows,
                    "sample_rows: add_prev must be a contiguous int32 [rows] tensor");
        TORCH_CHECK(logits_prev.has_value(), "sample_rows: add_prev needs logits_prev");
        a.add_prev = static_cast<const int32_t*>(add_prev->data_ptr());
    }
    if (uniforms.has_value()) {
        d.see(*uniforms);
        TORCH_CHECK(uniforms->scalar_type() == at::kFloat && uniforms->is_contiguous() && uniforms->numel() == rows && tokens_out.has_value(),
                    "sample_rows: uniforms must be a contiguous float32 [rows] tensor, given together with tokens_out");
        d.see(*tokens_out);
        TORCH_CHECK(tokens_out->scalar_type() == at::kLong && tokens_out->is_contiguous() && tokens_out->numel() == rows,
                    "sample_rows: tokens_out must be a contiguous int64 [rows] tensor");
        a.uniforms = static_cast<const float*>(uniforms->data_ptr());
        a.tokens = static_cast<int64_t*>(tokens_out->data_ptr());
    }
    if (probs_out.has_value()) {
        d.see(*probs_out);
        TORCH_CHECK(probs_out->scalar_type() == at::kFloat && probs_out->dim() == 2 && probs_out->size(0) == rows && probs_out->size(1) == V &&
                        probs_out->stride(1) == 1,
                    "sample_rows: probs_out must be float32 [rows, V] with a contiguous inner dimension");
        a.probs = static_cast<float*>(probs_out->data_ptr());
        a.probs_row_stride = rows > 1 ? probs_out->stride(0) : V;
    }
    TORCH_CHECK(a.tokens || a.probs, "sample_rows: nothing to produce (give uniforms and tokens_out, or probs_out)");
    if (row_enable.has_value()) {
        d.see(*row_enable);
        TORCH_CHECK((row_enable->scalar_type() == at::kBool || row_enable->scalar_type() == at::kByte) && row_enable->is_contiguous() &&
                        row_enable->numel() == rows,
                    "sample_rows: row_enable must be a contiguous bool/uint8 [rows] tensor");
        a.row_enable = static_cast<const uint8_t*>(row_enable->data_ptr());
    }
    a.rows = (int32_t)rows; a.vocab = (int32_t)V;
    a.temperature = (float)temperature; a.top_p = (float)top_p; a.min_p = (float)min_p;
    check_rc(g.sample_rows(&a, d.stream()), "tah_sample_rows");
}

Tensor silu_mul(const Tensor& gate_up, const optional<Tensor>& norm_input, double norm_eps) {
    need_lib();
    Dev d; d.see(gate_up); d.see(norm_input);
    TORCH_CHECK(gate_up.dim() == 2 && gate_up.scalar_type() == at::kBFloat16 && gate_up.size(1) % 16 == 0 && gate_up.stride(1) == 1,
                "silu_mul: gate_up must be bf16 [rows, 2*I] with I a multiple of 8 and a contiguous inner dimension");
    const int64_t rows = gate_up.size(0), inter = gate_up.size(1) / 2;
    auto out = at::empty({rows, inter}, gate_up.options());
    if (norm_input.has_value()) {
        TORCH_CHECK(norm_input->dim() == 2 && norm_input->scalar_type() == at::kBFloat16 && norm_input->size(0) == rows &&
                        norm_input->stride(1) == 1,
                    "silu_mul: norm_input must be a bf16 [rows, hidden] tensor with unit inner stride");
        check_rc(g.silu_mul_normed(ptr(gate_up), mptr(out), (int32_t)rows, (int32_t)inter, rows > 1 ? gate_up.stride(0) : 2 * inter, inter,
                                   ptr(*norm_input), rows > 1 ? norm_input->stride(0) : norm_input->size(1), (int32_t)norm_input->size(1),
                                   (float)norm_eps, d.stream()),
                 "tah_silu_mul_normed");
        return out;
    }
    check_rc(g.silu_mul(ptr(gate_up), mptr(out), (int32_t)rows, (int32_t)inter, rows > 1 ? gate_up.stride(0) : 2 * inter, inter, d.stream()),
             "tah_silu_mul");
    return out;
}

// Arg-max of the step's final logits and the generation loop's per-row bookkeeping, in place (tah_greedy_step).
void greedy_step(const Tensor& logits0, const optional<Tensor>& logits1, const optional<Tensor>& hard, int64_t eos, const Tensor& tok,
                 const Tensor& finished, const Tensor& pos, const Tensor& out_tokens, const Tensor& step_idx, const Tensor& out_len,
                 const Tensor& n_hard, const Tensor& n_steps) {
    need_lib();
    Dev d;
    for (const Tensor* t : {&logits0, &tok, &finished, &pos, &out_tokens, &step_idx, &out_len, &n_hard, &n_steps}) d.see(*t);
    d.see(logits1); d.see(hard);
    const int64_t rows = logits0.size(0), vocab = logits0.size(1);
    TORCH_CHECK(logits0.dim() == 2 && logits0.scalar_type() == at::kBFloat16 && logits0.stride(1) == 1, "greedy_step: logits0 must be bf16 [rows, vocab]");
    TORCH_CHECK(logits1.has_value() == hard.has_value(), "greedy_step: logits1 and hard come together");
    if (logits1.has_value()) {
        TORCH_CHECK(logits1->sizes() == logits0.sizes() && logits1->scalar_type() == at::kBFloat16 && logits1->stride(1) == 1,
                    "greedy_step: logits1 must match logits0");
        TORCH_CHECK(hard->scalar_type() == at::kBool && hard->is_contiguous() && hard->numel() == rows, "greedy_step: hard must be bool [rows]");
    }
    TORCH_CHECK(tok.scalar_type() == at::kLong && tok.is_contiguous() && tok.numel() == rows, "greedy_step: tok must be int64 [rows]");
    TORCH_CHECK(finished.scalar_type() == at::kBool && finished.is_contiguous() && finished.numel() == rows, "greedy_step: finished must be bool [rows]");
    TORCH_CHECK(pos.scalar_type() == at::kInt && pos.is_contiguous() && pos.numel() == rows, "greedy_step: pos must be int32 [rows]");
    TORCH_CHECK(out_len.scalar_type() == at::kInt && out_len.is_contiguous() && out_len.numel() == rows, "greedy_step: out_len must be int32 [rows]");
    TORCH_CHECK(out_tokens.scalar_type() == at::kLong && out_tokens.dim() == 2 && out_tokens.size(0) == rows && out_tokens.stride(1) == 1,
                "greedy_step: out_tokens must be int64 [rows, steps]");
    for (const Tensor* t : {&step_idx, &n_hard, &n_steps})
        TORCH_CHECK(t->scalar_type() == at::kLong && t->numel() == 1, "greedy_step: step_idx, n_hard and n_steps are int64 scalars");
    tah_greedy_step_args a{};
    a.logits0 = logits0.data_ptr(); a.logits1 = ptr(logits1); a.hard = static_cast<const uint8_t*>(ptr(hard));
    a.row_stride0 = logits0.stride(0); a.row_stride1 = logits1.has_value() ? logits1->stride(0) : 0;
    a.rows = (int32_t)rows; a.vocab = (int32_t)vocab; a.eos = (int32_t)eos;
    a.tok = static_cast<int64_t*>(tok.data_ptr()); a.finished = static_cast<uint8_t*>(finished.data_ptr());
    a.pos = static_cast<int32_t*>(pos.data_ptr()); a.out_tokens = static_cast<int64_t*>(out_tokens.data_ptr());
    a.out_stride = out_tokens.stride(0); a.step_idx = static_cast<const int64_t*>(step_idx.data_ptr());
    a.out_cols = (int32_t)out_tokens.size(1);
    a.out_len = static_cast<int32_t*>(out_len.data_ptr());
    a.n_hard = static_cast<int64_t*>(n_hard.data_ptr()); a.n_steps = static_cast<int64_t*>(n_steps.data_ptr());
    check_rc(g.greedy_step(&a, d.stream()), "tah_greedy_step");
}

// ---- glue of a generation step ---------------------------------------------------------------------------
bool vec_of(const Tensor& t, at::ScalarType ty, int64_t n) { return t.scalar_type() == ty && t.is_contiguous() && t.numel() == n; }

// tah_step_begin: everything a step needs before its first layer, written into the caller's tensors.
void step_begin(const Tensor& tok, const Tensor& pos, const Tensor& finished, const Tensor& embed, const Tensor& cos_table,
                const Tensor& sin_table, const Tensor& x, const optional<Tensor>& x_packed, const Tensor& cos_rows,
                const Tensor& sin_rows, const Tensor& slot, const Tensor& q_pos, const Tensor& active, const optional<Tensor>& phase,
                const optional<Tensor>& x_alt, const optional<Tensor>& hard_len, const optional<Tensor>& q_depth,
                const optional<Tensor>& append_at, const optional<Tensor>& eligible) {
    need_lib();
    Dev d;
    for (const Tensor* t : {&tok, &pos, &finished, &embed, &cos_table, &sin_table, &x, &cos_rows, &sin_rows, &slot, &q_pos, &active}) d.see(*t);
    d.see(x_packed); d.see(phase); d.see(x_alt); d.see(hard_len); d.see(q_depth); d.see(append_at); d.see(eligible);
    const int64_t rows = tok.numel(), hidden = embed.size(1);
    TORCH_CHECK(vec_of(tok, at::kLong, rows) && vec_of(pos, at::kInt, rows) && vec_of(finished, at::kBool, rows) &&
                    vec_of(slot, at::kInt, rows) && vec_of(q_pos, at::kInt, rows) && vec_of(active, at::kBool, rows),
                "step_begin: tok int64, pos / slot / q_pos int32, finished / active bool, all [rows]");
    TORCH_CHECK(embed.dim() == 2 && embed.scalar_type() == at::kBFloat16 && embed.stride(1) == 1, "step_begin: embed must be bf16 [V, H]");
    for (const Tensor* t : {&cos_table, &sin_table})
        TORCH_CHECK(t->dim() == 2 && t->size(1) == 128 && t->scalar_type() == at::kBFloat16 && t->is_contiguous() && t->size(0) == cos_table.size(0),
                    "step_begin: the rotary tables must be contiguous bf16 [L, 128]");
    TORCH_CHECK(x.dim() == 2 && x.size(0) == rows && x.size(1) == hidden && x.scalar_type() == at::kBFloat16 && (rows == 0 || x.stride(1) == 1),
                "step_begin: x must be bf16 [rows, H]");
    for (const Tensor* t : {&cos_rows, &sin_rows}) TORCH_CHECK(vec_of(*t, at::kBFloat16, rows * 128), "step_begin: cos_rows / sin_rows must be contiguous bf16 [rows, 128]");
    if (x_packed.has_value()) TORCH_CHECK(vec_of(*x_packed, at::kBFloat16, 32 * hidden), "step_begin: x_packed must be a contiguous bf16 tensor of 32 * H elements");
    tah_step_begin_args a{};
    a.tok = static_cast<const int64_t*>(tok.data_ptr()); a.pos = static_cast<const int32_t*>(pos.data_ptr());
    a.finished = static_cast<const uint8_t*>(finished.data_ptr());
    a.embed = embed.data_ptr(); a.embed_row_stride = embed.stride(0);
    a.cos_table = cos_table.data_ptr(); a.sin_table = sin_table.data_ptr();
    a.rows = (int32_t)rows; a.vocab = (int32_t)embed.size(0); a.hidden = (int32_t)hidden; a.table_rows = (int32_t)cos_table.size(0);
    a.x = x.data_ptr(); a.x_row_stride = rows > 1 ? x.stride(0) : hidden;
    a.x_packed = x_packed.has_value() ? x_packed->data_ptr() : nullptr;
    a.cos_rows = cos_rows.data_ptr(); a.sin_rows = sin_rows.data_ptr();
    a.slot = static_cast<int32_t*>(slot.data_ptr()); a.q_pos = static_cast<int32_t*>(q_pos.data_ptr());
    a.active = static_cast<uint8_t*>(active.data_ptr());
    for (const optional<Tensor>* t : {&phase, &hard_len, &q_depth, &append_at})
        if (t->has_value()) TORCH_CHECK(vec_of(**t, at::kInt, rows), "step_begin: phase, hard_len, q_depth and append_at are int32 [rows]");
    if (eligible.has_value()) TORCH_CHECK(vec_of(*eligible, at::kBool, rows), "step_begin: eligible must be bool [rows]");
    if (x_alt.has_value())
        TORCH_CHECK(x_alt->dim() == 2 && x_alt->size(0) == rows && x_alt->size(1) == hidden && x_alt->scalar_type() == at::kBFloat16 &&
                        (rows == 0 || x_alt->stride(1) == 1),
                    "step_begin: x_alt must be bf16 [rows, H]");
    a.phase = phase.has_value() ? static_cast<const int32_t*>(phase->data_ptr()) : nullptr;
    a.x_alt = x_alt.has_value() ? x_alt->data_ptr() : nullptr;
    a.x_alt_row_stride = x_alt.has_value() ? (rows > 1 ? x_alt->stride(0) : hidden) : 0;
    a.hard_len = hard_len.has_value() ? static_cast<const int32_t*>(hard_len->data_ptr()) : nullptr;
    a.q_depth = q_depth.has_value() ? static_cast<int32_t*>(q_depth->data_ptr()) : nullptr;
    a.append_at = append_at.has_value() ? static_cast<int32_t*>(append_at->data_ptr()) : nullptr;
    a.eligible = eligible.has_value() ? static_cast<uint8_t*>(eligible->data_ptr()) : nullptr;
    check_rc(g.step_begin(&a, d.stream()), "tah_step_begin");
}

// tah_greedy_tick: tokens and bookkeeping at the end of a tick whose rows are at different latent iterations.
void greedy_tick(const Tensor& logits, const Tensor& logits_prev, int64_t eos, int64_t limit, const Tensor& hard_now, const Tensor& phase,
                 const Tensor& tok, const Tensor& finished, const Tensor& pos, const Tensor& out_tokens, const Tensor& out_len,
                 const Tensor& hard_len, const Tensor& n_hard, const Tensor& n_steps, const optional<Tensor>& chosen) {
    need_lib();
    Dev d;
    for (const Tensor* t : {&logits, &logits_prev, &hard_now, &phase, &tok, &finished, &pos, &out_tokens, &out_len, &hard_len, &n_hard, &n_steps}) d.see(*t);
    d.see(chosen);
    const int64_t rows = logits.size(0), vocab = logits.size(1);
    for (const Tensor* t : {&logits, &logits_prev})
        TORCH_CHECK(t->dim() == 2 && t->size(0) == rows && t->size(1) == vocab && t->scalar_type() == at::kBFloat16 && t->stride(1) == 1,
                    "greedy_tick: logits and logits_prev must be bf16 [rows, vocab]");
    TORCH_CHECK(vec_of(hard_now, at::kBool, rows) && vec_of(finished, at::kBool, rows), "greedy_tick: hard_now and finished are bool [rows]");
    for (const Tensor* t : {&phase, &pos, &out_len, &hard_len}) TORCH_CHECK(vec_of(*t, at::kInt, rows), "greedy_tick: phase, pos, out_len and hard_len are int32 [rows]");
    TORCH_CHECK(vec_of(tok, at::kLong, rows), "greedy_tick: tok must be int64 [rows]");
    TORCH_CHECK(out_tokens.scalar_type() == at::kLong && out_tokens.dim() == 2 && out_tokens.size(0) == rows && out_tokens.stride(1) == 1 &&
                    out_tokens.size(1) >= limit,
                "greedy_tick: out_tokens must be int64 [rows, >= limit]");
    for (const Tensor* t : {&n_hard, &n_steps}) TORCH_CHECK(t->scalar_type() == at::kLong && t->numel() == 1, "greedy_tick: n_hard and n_steps are int64 scalars");
    tah_greedy_tick_args a{};
    a.logits = logits.data_ptr(); a.logits_prev = logits_prev.data_ptr();
    a.row_stride = rows > 1 ? logits.stride(0) : vocab; a.row_stride_prev = rows > 1 ? logits_prev.stride(0) : vocab;
    a.rows = (int32_t)rows; a.vocab = (int32_t)vocab; a.eos = (int32_t)eos; a.limit = (int32_t)limit;
    a.hard_now = static_cast<const uint8_t*>(hard_now.data_ptr()); a.phase = static_cast<int32_t*>(phase.data_ptr());
    a.tok = static_cast<int64_t*>(tok.data_ptr()); a.finished = static_cast<uint8_t*>(finished.data_ptr());
    a.pos = static_cast<int32_t*>(pos.data_ptr()); a.out_tokens = static_cast<int64_t*>(out_tokens.data_ptr());
    a.out_stride = out_tokens.stride(0); a.out_len = static_cast<int32_t*>(out_len.data_ptr());
    a.hard_len = static_cast<int32_t*>(hard_len.data_ptr());
    a.n_hard = static_cast<int64_t*>(n_hard.data_ptr()); a.n_steps = static_cast<int64_t*>(n_steps.data_ptr());
    if (chosen.has_value()) {
        TORCH_CHECK(vec_of(*chosen, at::kLong, rows), "greedy_tick: chosen must be int64 [rows]");
        a.chosen = static_cast<const int64_t*>(chosen->data_ptr());
    }
    check_rc(g.greedy_tick(&a, d.stream()), "tah_greedy_tick");
}

// tah_decider_tail: second layer of the decider, the decision, and the second iteration's per-row bookkeeping.
void decider_tail(const Tensor& hidden, const Tensor& w2, const optional<Tensor>& b2, double threshold, const optional<Tensor>& active,
                  const optional<Tensor>& pos, const Tensor& hard, const optional<Tensor>& hard_i32, const optional<Tensor>& slot,
                  const optional<Tensor>& q_pos) {
    need_lib();
    Dev d; d.see(hidden); d.see(w2); d.see(b2); d.see(active); d.see(pos); d.see(hard); d.see(hard_i32); d.see(slot); d.see(q_pos);
    TORCH_CHECK(hidden.dim() == 2 && hidden.scalar_type() == at::kBFloat16 && (hidden.numel() == 0 || hidden.stride(1) == 1), "decider_tail: hidden must be bf16 [rows, width]");
    const int64_t rows = hidden.size(0), width = hidden.size(1);
    TORCH_CHECK(vec_of(w2, at::kBFloat16, width), "decider_tail: w2 must be a contiguous bf16 tensor of `width` elements");
    if (b2.has_value()) TORCH_CHECK(vec_of(*b2, at::kBFloat16, 1), "decider_tail: b2 must be a bf16 scalar");
    TORCH_CHECK(vec_of(hard, at::kBool, rows), "decider_tail: hard must be bool [rows]");
    if (active.has_value()) TORCH_CHECK(vec_of(*active, at::kBool, rows), "decider_tail: active must be bool [rows]");
    for (const optional<Tensor>* t : {&pos, &hard_i32, &slot, &q_pos})
        if (t->has_value()) TORCH_CHECK(vec_of(**t, at::kInt, rows), "decider_tail: pos, hard_i32, slot and q_pos are int32 [rows]");
    tah_decider_tail_args a{};
    a.hidden = hidden.data_ptr(); a.hidden_row_stride = rows > 1 ? hidden.stride(0) : width;
    a.w2 = w2.data_ptr(); a.b2 = b2.has_value() ? b2->data_ptr() : nullptr;
    a.threshold = (float)threshold; a.rows = (int32_t)rows; a.width = (int32_t)width;
    a.active = active.has_value() ? static_cast<const uint8_t*>(active->data_ptr()) : nullptr;
    a.pos = pos.has_value() ? static_cast<const int32_t*>(pos->data_ptr()) : nullptr;
    a.hard = static_cast<uint8_t*>(hard.data_ptr());
    a.hard_i32 = hard_i32.has_value() ? static_cast<int32_t*>(hard_i32->data_ptr()) : nullptr;
    a.slot = slot.has_value() ? static_cast<int32_t*>(slot->data_ptr()) : nullptr;
    a.q_pos = q_pos.has_value() ? static_cast<int32_t*>(q_pos->data_ptr()) : nullptr;
    check_rc(g.decider_tail(&a, d.stream()), "tah_decider_tail");
}

// ---- linear layers of a decode step (tah_linear_rows) ------------------------------------------------------
bool packed_vec(const Tensor& t, int64_t numel) {
    return t.scalar_type() == at::kBFloat16 && t.is_contiguous() && t.numel() == numel;
}

// w [n, k] (gate_up: [2 n, k], gate rows then up rows) -> the weight in the order tah_linear_rows reads it, [n * k] or [2 n * k]
Tensor linear_pack_weight(const Tensor& w, bool gate_up) {
    need_lib();
    Dev d; d.see(w);
    TORCH_CHECK(w.dim() == 2 && w.scalar_type() == at::kBFloat16 && w.stride(1) == 1, "linear_pack_weight: w must be a bf16 [N, K] matrix");
    TORCH_CHECK(!gate_up || w.size(0) % 2 == 0, "linear_pack_weight: a stacked [gate; up] weight has an even number of rows");
    const int64_t n = gate_up ? w.size(0) / 2 : w.size(0), k = w.size(1);
    Tensor out = at::empty({w.size(0) * k}, w.options());
    check_rc(g.linear_pack_weight(ptr(w), w.stride(0), mptr(out), (int32_t)n, (int32_t)k, gate_up ? TAH_LINEAR_GATE_UP : TAH_LINEAR_PLAIN, d.stream()),
             "tah_linear_pack_weight");
    return out;
}

// x [rows <= 32, k] -> packed rows [32 * k]
Tensor linear_pack_rows(const Tensor& x, const optional<Tensor>& out) {
    need_lib();
    Dev d; d.see(x); d.see(out);
    TORCH_CHECK(x.dim() == 2 && x.scalar_type() == at::kBFloat16 && (x.numel() == 0 || x.stride(1) == 1), "linear_pack_rows: x must be a bf16 [rows, K] matrix");
    const int64_t rows = x.size(0), k = x.size(1);
    Tensor xp = out.has_value() ? *out : at::empty({32 * k}, x.options());
    TORCH_CHECK(packed_vec(xp, 32 * k), "linear_pack_rows: out must be a contiguous bf16 tensor of 32 * K elements");
    check_rc(g.linear_pack_rows(ptr(x), rows > 1 ? x.stride(0) : k, mptr(xp), (int32_t)rows, (int32_t)k, d.stream()), "tah_linear_pack_rows");
    return xp;
}

// out = x W^T [+ residual] or silu(gate) * up, from packed operands; returns the row-major result (or nothing when
// only the packed result is asked for).
optional<Tensor> linear_rows(const Tensor& w_packed, const Tensor& x_packed, int64_t rows, int64_t n, int64_t k, bool gate_up,
                             const optional<Tensor>& residual, const optional<Tensor>& out, const optional<Tensor>& out_packed,
                             bool want_out, int64_t input_norm, double norm_eps, const optional<Tensor>& bias, int64_t activation,
                             const optional<Tensor>& ln_colsum) {
    need_lib();
    Dev d; d.see(w_packed); d.see(x_packed); d.see(residual); d.see(out); d.see(out_packed); d.see(bias); d.see(ln_colsum);
    if (ln_colsum.has_value())
        TORCH_CHECK(ln_colsum->scalar_type() == at::kFloat && ln_colsum->is_contiguous() && ln_colsum->numel() == n,
                    "linear_rows: ln_colsum must be a contiguous float32 [N] tensor");
    TORCH_CHECK((input_norm == TAH_NORM_LAYER) == ln_colsum.has_value(), "linear_rows: ln_colsum goes with the LayerNorm fold and only with it");
    if (bias.has_value()) TORCH_CHECK(packed_vec(*bias, n), "linear_rows: bias must be a contiguous bf16 [N] tensor");
    TORCH_CHECK(rows >= 0 && n >= 0 && k >= 0, "linear_rows: negative size");
    TORCH_CHECK(packed_vec(w_packed, (gate_up ? 2 : 1) * n * k), "linear_rows: w_packed must come from linear_pack_weight for these sizes");
    TORCH_CHECK(packed_vec(x_packed, 32 * k), "linear_rows: x_packed must be a contiguous bf16 tensor of 32 * K elements");
    optional<Tensor> y = out;
    if (!y.has_value() && want_out) y = at::empty({rows, n}, x_packed.options());
    if (y.has_value())
        TORCH_CHECK(y->dim() == 2 && y->size(0) == rows && y->size(1) == n && y->scalar_type() == at::kBFloat16 && (y->numel() == 0 || y->stride(1) == 1),
                    "linear_rows: out must be bf16 [rows, N]");
    if (residual.has_value())
        TORCH_CHECK(residual->dim() == 2 && residual->size(0) == rows && residual->size(1) == n && residual->scalar_type() == at::kBFloat16 &&
                        (residual->numel() == 0 || residual->stride(1) == 1),
                    "linear_rows: residual must be bf16 [rows, N]");
    if (out_packed.has_value()) TORCH_CHECK(packed_vec(*out_packed, 32 * n), "linear_rows: out_packed must be a contiguous bf16 tensor of 32 * N elements");
    TORCH_CHECK(y.has_value() || out_packed.has_value(), "linear_rows: nothing to write");
    tah_linear_rows_args a{};
    a.w_packed = w_packed.data_ptr(); a.x_packed = x_packed.data_ptr();
    a.residual = ptr(residual); a.residual_row_stride = residual.has_value() ? (rows > 1 ? residual->stride(0) : n) : 0;
    a.out = y.has_value() ? mptr(*y) : nullptr; a.out_row_stride = y.has_value() ? (rows > 1 ? y->stride(0) : n) : 0;
    a.out_packed = out_packed.has_value() ? out_packed->data_ptr() : nullptr;
    a.rows = (int32_t)rows; a.n = (int32_t)n; a.k = (int32_t)k;
    a.kind = gate_up ? TAH_LINEAR_GATE_UP : TAH_LINEAR_PLAIN;
    a.input_norm = (int32_t)input_norm; a.norm_eps = (float)norm_eps;
    a.bias = bias.has_value() ? bias->data_ptr() : nullptr; a.activation = (int32_t)activation;
    a.ln_colsum = ln_colsum.has_value() ? static_cast<const float*>(ln_colsum->data_ptr()) : nullptr;
    check_rc(g.linear_rows(&a, d.stream()), "tah_linear_rows");
    return y;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "PyTorch-ROCm binding of the duo-causal attention C ABI (include/tah_duo.h)";
    m.def("load_library", &load_library, py::arg("path"), py::arg("allow_host") = false);
    m.def("loaded", [] { return g.handle != nullptr; });
    m.def("abi_version", [] { need_lib(); return g.abi_version(); });
    m.def("duo_schedule", &duo_schedule);
    m.def("greedy_step", &greedy_step);
    m.def("duo_fwd_varlen", &duo_fwd_varlen);
    m.def("duo_bwd_varlen", &duo_bwd_varlen);
    m.def("duo_bwd_workspace_bytes", [](int64_t nseq, int64_t hq, int64_t hkv, int64_t tq1, int64_t tk1, int64_t tq2, int64_t tk2,
                                        int64_t mk1, int64_t mk2) {
        need_lib();
        return (int64_t)g.bwd_workspace_bytes((int32_t)nseq, (int32_t)hq, (int32_t)hkv, (int32_t)tq1, (int32_t)tk1, (int32_t)tq2,
                                              (int32_t)tk2, (int32_t)mk1, (int32_t)mk2);
    });
    m.def("duo_fwd_masked", &duo_fwd_masked);
    m.def("duo_bwd_masked", &duo_bwd_masked);
    m.def("decode_workspace_bytes", &decode_workspace_bytes);
    m.def("duo_decode", &duo_decode);
    m.def("kv_append", &kv_append);
    m.def("qk_prep", &qk_prep);
    m.def("hard_index_build", &hard_index_build);
    m.def("pad_rows_build", &pad_rows_build);
    m.def("rows_copy", &rows_copy);
    m.def("topk_mix", &topk_mix);
    m.def("sample_rows", &sample_rows);
    m.def("qk_prep_bwd", &qk_prep_bwd);
    m.def("topk_values", &topk_values);
    m.def("silu_mul", &silu_mul);
    m.def("duo_decode_step", &duo_decode_step);
    m.def("duo_decode_step_supported", &duo_decode_step_supported);
    m.def("step_begin", &step_begin);
    m.def("greedy_tick", &greedy_tick);
    m.def("decider_tail", &decider_tail);
    m.def("linear_pack_weight", &linear_pack_weight);
    m.def("linear_pack_rows", &linear_pack_rows);
    m.def("linear_rows", &linear_rows);
}
