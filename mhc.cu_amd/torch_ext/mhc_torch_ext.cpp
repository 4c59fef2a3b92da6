// PyTorch-ROCm extension over the C ABI of libmhc_hip.so: allocates outputs, passes raw device
// pointers and torch's current HIP stream, and implements the autograd functions in C++.
//
// Counterpart of the reference's pybind module `mhc_cuda` (src/python/bindings.cu:544-554) and of
// the autograd classes of src/python/mhc/ops.py:13-417.  No torch type crosses into the library:
// every mhc_* call below is the C ABI of include/mhc_hip.h.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <mutex>
#include <unordered_map>

#include "../../include/mhc_hip.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;
using OptTensor = c10::optional<Tensor>;

struct MhcError : std::runtime_error {
    std::string fn;
    int status;
    MhcError(const char *f, int s)
        : std::runtime_error(std::string(f) + " failed: " + mhc_status_string(s) + " (status " + std::to_string(s) + ")"),
          fn(f), status(s) {}
};

inline void check(const char *fn, int status) {
    if (status != MHC_OK) throw MhcError(fn, status);
}

inline int dt(const Tensor &t) {
    if (t.scalar_type() == at::kFloat) return MHC_F32;
    if (t.scalar_type() == at::kBFloat16) return MHC_BF16;
    TORCH_CHECK(false, "mhc: unsupported dtype ", t.scalar_type(), ": the HIP library takes float32 or bfloat16");
}
inline bool is_act_dtype(const Tensor &t) { return t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16; }

inline void *ptr(const Tensor &t) { return t.defined() ? t.data_ptr() : nullptr; }

inline void require_gpu(const Tensor &t) {
    if (!t.defined()) return;
    TORCH_CHECK(t.is_cuda(), "mhc: tensors must live on a HIP (cuda) device; there is no CPU path");
}

// contiguous, on the device, and with a 16-byte aligned base (a contiguous view at an odd offset is copied)
inline Tensor act(const Tensor &t) {
    require_gpu(t);
    Tensor c = t.contiguous();
    if ((reinterpret_cast<uintptr_t>(c.data_ptr()) & 15u) != 0) c = c.clone();
    return c;
}
inline Tensor f32c(const Tensor &t) {
    require_gpu(t);
    return (t.scalar_type() == at::kFloat ? t : t.to(at::kFloat)).contiguous();
}

inline void *stream_of(const Tensor &t) {
    return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

// Scratch buffer per (device, stream), grown on demand.  Kernels that use it are ordered on that
// stream, so reuse across calls is safe.
Tensor workspace(const Tensor &like, size_t nbytes) {
    static std::mutex mu;
    static std::unordered_map<uint64_t, Tensor> cache;
    const uint64_t key = (static_cast<uint64_t>(like.device().index()) << 56) ^
                         reinterpret_cast<uint64_t>(stream_of(like));
    std::lock_guard<std::mutex> lock(mu);
    auto it = cache.find(key);
    if (it == cache.end() || static_cast<size_t>(it->second.numel()) < nbytes) {
        const int64_t want = static_cast<int64_t>(std::max<size_t>(nbytes, 1 << 20));
        Tensor buf = at::empty({want}, like.options().dtype(at::kByte));
        cache[key] = buf;
        return buf;
    }
    return it->second;
}

// ---------------------------------------------------------------------------------------------
// parameter packing (dynamic H): phi [D, nC] in the compute dtype, bias | alpha as one fp32 [D+3]
// ---------------------------------------------------------------------------------------------
struct Packed {
    Tensor phi, ba;  // ba = [bias (D) | alpha (3)]
};

bool g_param_cache = false;

// An entry is valid while the very same tensor objects are alive (weak references: a new tensor that
// happens to reuse the address of a freed one never matches) and their storage addresses and
// in-place version counters are unchanged.
struct CacheEntry {
    c10::weak_intrusive_ptr<c10::TensorImpl> impl[9];
    void *ptrs[9];
    uint32_t versions[9];
    int cd;
    Packed packed;
    CacheEntry()
        : impl{c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>()),
               c10::weak_intrusive_ptr<c10::TensorImpl>(c10::intrusive_ptr<c10::TensorImpl>())} {}
};

Packed pack_params(const Tensor &phi_pre, const Tensor &phi_post, const Tensor &phi_res, const Tensor &alpha_pre,
                   const Tensor &alpha_post, const Tensor &alpha_res, const Tensor &b_pre, const Tensor &b_post,
                   const Tensor &b_res, int n, int C, at::ScalarType compute) {
    static std::mutex mu;
    static std::unordered_map<void *, CacheEntry> cache;
    const Tensor *src[9] = {&phi_pre, &phi_post, &phi_res, &alpha_pre, &alpha_post, &alpha_res, &b_pre, &b_post, &b_res};
    const int cd = compute == at::kBFloat16 ? MHC_BF16 : MHC_F32;
    if (g_param_cache) {
        std::lock_guard<std::mutex> lock(mu);
        auto it = cache.find(phi_pre.data_ptr());
        if (it != cache.end() && it->second.cd == cd) {
            bool same = true;
            for (int i = 0; i < 9; i++)
                same = same && !it->second.impl[i].expired() &&
                       it->second.impl[i]._unsafe_get_target() == src[i]->unsafeGetTensorImpl() &&
                       it->second.ptrs[i] == src[i]->data_ptr() && it->second.versions[i] == src[i]->_version();
            if (same) return it->second.packed;
        }
    }
    const int D = n * n + 2 * n;
    // the three phi matrices in one source dtype the kernel reads (float32 or bfloat16)
    const bool same_dt = phi_pre.scalar_type() == phi_post.scalar_type() && phi_pre.scalar_type() == phi_res.scalar_type() &&
                         is_act_dtype(phi_pre);
    const Tensor pp = same_dt ? phi_pre.contiguous() : f32c(phi_pre);
    const Tensor po = same_dt ? phi_post.contiguous() : f32c(phi_post);
    const Tensor pr = same_dt ? phi_res.contiguous() : f32c(phi_res);
    for (const Tensor *t : {&pp, &po, &pr}) require_gpu(*t);
    const Tensor bp = f32c(b_pre), bo = f32c(b_post), br = f32c(b_res);
    const Tensor ap = f32c(alpha_pre), ao = f32c(alpha_post), ar = f32c(alpha_res);
    TORCH_CHECK(pp.numel() == (int64_t)n * n * C && po.numel() == pp.numel() && pr.numel() == (int64_t)n * n * n * C,
                "mhc: phi shapes do not match expansion rate ", n, " and hidden size ", C);
    TORCH_CHECK(bp.numel() == n && bo.numel() == n && br.numel() == n * n, "mhc: bias shapes do not match n = ", n);
    Packed out;
    out.phi = at::empty({D, (int64_t)n * C}, pp.options().dtype(compute));
    out.ba = at::empty({D + 3}, pp.options().dtype(at::kFloat));
    check("mhc_pack_dynamic_params",
          mhc_pack_dynamic_params(ptr(pp), ptr(po), ptr(pr), dt(pp), bp.data_ptr<float>(), bo.data_ptr<float>(),
                                  br.data_ptr<float>(), ap.data_ptr<float>(), ao.data_ptr<float>(),
                                  ar.data_ptr<float>(), ptr(out.phi), cd, out.ba.data_ptr<float>(),
                                  out.ba.data_ptr<float>() + D, n, C, stream_of(pp)));
    if (g_param_cache) {
        std::lock_guard<std::mutex> lock(mu);
        if (cache.size() >= 4096) cache.clear();
        CacheEntry e;
        for (int i = 0; i < 9; i++) {
            e.impl[i] = c10::weak_intrusive_ptr<c10::TensorImpl>(src[i]->getIntrusivePtr());
            e.ptrs[i] = src[i]->data_ptr();
            e.versions[i] = src[i]->_version();
        }
        e.cd = cd;
        e.packed = out;
        cache.erase(phi_pre.data_ptr());
        cache.emplace(phi_pre.data_ptr(), std::move(e));
    }
    return out;
}

// ---------------------------------------------------------------------------------------------
// dynamic-H layer (reference ops.py:154-417, bindings.cu:405-542)
// ---------------------------------------------------------------------------------------------
struct DynFwdOut {
    Tensor y, small;  // small = fp32: Hpre | Hpost | M | P | r | q | Sinkhorn state, B * (2n + n*n + D + 2) + state floats
};

struct SmallViews {
    float *Hp, *Ho, *M, *P, *r, *q, *sk;
    static int64_t coef_floats(int B, int n) { return (int64_t)B * (2 * n + n * n + (n * n + 2 * n) + 2); }
    SmallViews(const Tensor &small, int B, int n) {
        const int D = n * n + 2 * n;
        float *b = small.data_ptr<float>();
        Hp = b; Ho = Hp + (size_t)B * n; M = Ho + (size_t)B * n; P = M + (size_t)B * n * n;
        r = P + (size_t)B * D; q = r + B;
        sk = small.numel() > coef_floats(B, n) ? q + B : nullptr;  // present when the forward ran under autograd
    }
};

DynFwdOut dyn_forward(const Tensor &x, int x_code, const OptTensor &w, const Packed &pk, const OptTensor &f_inject,
                      at::ScalarType out_dtype, int iters, double eps, bool for_backward) {
    const int B = x.size(0), n = x.size(1), C = x.size(2), D = n * n + 2 * n;
    c10::DeviceGuard guard(x.device());
    DynFwdOut o;
    o.y = at::empty({B, n, C}, x.options().dtype(out_dtype));
    // the Sinkhorn denominators are only worth writing when a backward call will read them
    const int64_t state = for_backward ? (int64_t)mhc_layer_sinkhorn_state_floats(B, n, iters) : 0;
    o.small = at::empty({SmallViews::coef_floats(B, n) + state}, x.options().dtype(at::kFloat));
    SmallViews v(o.small, B, n);
    const size_t need = mhc_layer_dynamic_workspace_bytes(B, n, C);
    Tensor ws = workspace(x, need);
    const Tensor wt = w.has_value() ? *w : Tensor();
    const Tensor ft = f_inject.has_value() ? *f_inject : Tensor();
    float *ba = pk.ba.data_ptr<float>();
    check("mhc_layer_fwd_dynamic",
          mhc_layer_fwd_dynamic(ptr(x), x_code, ptr(wt), wt.defined() ? dt(wt) : 0, ptr(pk.phi), dt(pk.phi), ba, ba + D,
                                ptr(ft), ptr(o.y), dt(o.y), v.Hp, v.Ho, v.M, v.P, v.r, v.q, v.sk, B, n, C, iters,
                                (float)eps, ws.data_ptr(), (size_t)ws.numel(), stream_of(x)));
    return o;
}

struct MHCDynamicFn : public torch::autograd::Function<MHCDynamicFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &x_in, const OptTensor &w_in, const Tensor &phi_pre,
                          const Tensor &phi_post, const Tensor &phi_res, const Tensor &alpha_pre,
                          const Tensor &alpha_post, const Tensor &alpha_res, const Tensor &b_pre, const Tensor &b_post,
                          const Tensor &b_res, int64_t iters, double eps, c10::optional<at::ScalarType> out_dtype,
                          const OptTensor &f_in, bool grad_mode, bool compute_bf16) {
        TORCH_CHECK(x_in.dim() == 3, "mhc: x must be [B, n, C]");
        // compute_bf16 with float32 activations (the reference's default contract: float32 in and out
        // around a bf16 kernel path): where the library's kernels load fp32 storage themselves, x is
        // handed over as it is and rounded in registers; elsewhere it is cast here, as the reference
        // casts it (bindings.cu:421-423)
        Tensor x = act(is_act_dtype(x_in) ? x_in : x_in.to(at::kFloat));
        const int B = x.size(0), n = x.size(1), C = x.size(2);
        int x_code = dt(x);
        if (compute_bf16 && x.scalar_type() == at::kFloat) {
            if (out_dtype.value_or(at::kFloat) == at::kFloat && mhc_layer_dynamic_accepts_f32_as_bf16(B, n, C, (int)iters))
                x_code = MHC_F32_AS_BF16;
            else {
                x = x.to(at::kBFloat16);
                x_code = MHC_BF16;
            }
        }
        OptTensor w, f;
        if (w_in.has_value() && w_in->defined()) w = act(is_act_dtype(*w_in) ? *w_in : w_in->to(at::kFloat));
        if (f_in.has_value() && f_in->defined()) f = act(f_in->to(x.scalar_type()));
        const Packed pk = pack_params(phi_pre, phi_post, phi_res, alpha_pre, alpha_post, alpha_res, b_pre, b_post, b_res,
                                      n, C, x_code == MHC_F32 ? at::kFloat : at::kBFloat16);
        DynFwdOut o = dyn_forward(x, x_code, w, pk, f, out_dtype.value_or(at::kFloat), (int)iters, eps, grad_mode);
        ctx->save_for_backward({x, w.has_value() ? *w : Tensor(), pk.phi, pk.ba, f.has_value() ? *f : Tensor(), o.small});
        ctx->saved_data["iters"] = iters;
        ctx->saved_data["eps"] = eps;
        ctx->saved_data["x_dtype"] = (int64_t)x_in.scalar_type();
        ctx->saved_data["x_code"] = (int64_t)x_code;
        ctx->saved_data["w_dtype"] = (int64_t)(w_in.has_value() && w_in->defined() ? w_in->scalar_type() : at::kFloat);
        ctx->saved_data["f_dtype"] = (int64_t)(f_in.has_value() && f_in->defined() ? f_in->scalar_type() : at::kFloat);
        ctx->saved_data["phi_dtypes"] = std::vector<int64_t>{(int64_t)phi_pre.scalar_type(), (int64_t)phi_post.scalar_type(),
                                                             (int64_t)phi_res.scalar_type()};
        ctx->saved_data["alpha_dtypes"] = std::vector<int64_t>{(int64_t)alpha_pre.scalar_type(), (int64_t)alpha_post.scalar_type(),
                                                               (int64_t)alpha_res.scalar_type()};
        ctx->saved_data["b_dtypes"] = std::vector<int64_t>{(int64_t)b_pre.scalar_type(), (int64_t)b_post.scalar_type(),
                                                           (int64_t)b_res.scalar_type()};
        ctx->saved_data["b_res_shape"] = b_res.sizes().vec();
        return o.y;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &x = saved[0], &w = saved[1], &phi = saved[2], &ba = saved[3], &f = saved[4], &small = saved[5];
        const int B = x.size(0), n = x.size(1), C = x.size(2), D = n * n + 2 * n;
        c10::DeviceGuard guard(x.device());
        const int iters = (int)ctx->saved_data["iters"].toInt();
        const double eps = ctx->saved_data["eps"].toDouble();
        // bfloat16 activations with a float32 result hand back a float32 gradient: it is rounded to the
        // activations' format here, so that the backward runs the kernels that take both in 2 bytes (the
        // mixed pair goes through slower general kernels: 111 against 20 us for dx at B=128 n=32 C=1280).
        // One pass also when the gradient arrives as a broadcast view (the backward of a sum).
        const bool round_dy = x.scalar_type() == at::kBFloat16 && grads[0].scalar_type() == at::kFloat;
        Tensor dy = act(round_dy ? grads[0].to(grads[0].options().dtype(at::kBFloat16), false, false, at::MemoryFormat::Contiguous)
                                 : grads[0]);
        const auto fo = x.options().dtype(at::kFloat);
        Tensor dx = at::empty_like(x);
        Tensor df = f.defined() ? at::empty_like(f) : Tensor();
        Tensor dw = f.defined() ? Tensor() : at::empty({C}, fo);
        Tensor dphi = at::empty({D, (int64_t)n * C}, fo);
        Tensor dba = at::empty({D + 3}, fo);
        SmallViews v(small, B, n);
        Tensor ws = workspace(x, mhc_layer_dynamic_workspace_bytes(B, n, C));
        float *bap = ba.data_ptr<float>();
        check("mhc_layer_bwd_dynamic",
              mhc_layer_bwd_dynamic(ptr(dy), dt(dy), ptr(x), (int)ctx->saved_data["x_code"].toInt(), ptr(w), w.defined() ? dt(w) : 0, ptr(phi), dt(phi), bap,
                                    bap + D, ptr(f), v.Hp, v.Ho, v.M, v.P, v.r, v.q, v.sk, ptr(dx), ptr(df),
                                    dw.defined() ? dw.data_ptr<float>() : nullptr, dphi.data_ptr<float>(),
                                    dba.data_ptr<float>(), dba.data_ptr<float>() + D, B, n, C, iters, (float)eps,
                                    ws.data_ptr(), (size_t)ws.numel(), stream_of(x)));
        auto to = [](const Tensor &t, int64_t st) {
            const auto s = (at::ScalarType)st;
            return t.scalar_type() == s ? t : t.to(s);
        };
        const auto pd = ctx->saved_data["phi_dtypes"].toIntVector();
        const auto ad = ctx->saved_data["alpha_dtypes"].toIntVector();
        const auto bd = ctx->saved_data["b_dtypes"].toIntVector();
        const auto brs = ctx->saved_data["b_res_shape"].toIntVector();
        variable_list out(17);
        out[0] = to(dx, ctx->saved_data["x_dtype"].toInt());
        out[1] = (dw.defined() && w.defined()) ? to(dw, ctx->saved_data["w_dtype"].toInt()) : Tensor();
        out[2] = to(dphi.narrow(0, 0, n), pd[0]);
        out[3] = to(dphi.narrow(0, n, n), pd[1]);
        out[4] = to(dphi.narrow(0, 2 * n, n * n), pd[2]);
        for (int i = 0; i < 3; i++) out[5 + i] = to(dba.select(0, D + i), ad[i]);
        out[8] = to(dba.narrow(0, 0, n), bd[0]);
        out[9] = to(dba.narrow(0, n, n), bd[1]);
        out[10] = to(dba.narrow(0, 2 * n, n * n).reshape(brs), bd[2]);
        out[14] = df.defined() ? to(df, ctx->saved_data["f_dtype"].toInt()) : Tensor();
        return out;
    }
};

// ---------------------------------------------------------------------------------------------
// static-H layer (reference ops.py:55-151, bindings.cu:221-401)
// ---------------------------------------------------------------------------------------------
struct MHCStaticFn : public torch::autograd::Function<MHCStaticFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &x_in, const OptTensor &w_in, const Tensor &H_pre,
                          const Tensor &H_post, const Tensor &H_res, int64_t iters, double eps,
                          c10::optional<at::ScalarType> out_dtype, const OptTensor &f_in) {
        TORCH_CHECK(x_in.dim() == 3, "mhc: x must be [B, n, C]");
        const Tensor x = act(is_act_dtype(x_in) ? x_in : x_in.to(at::kFloat));
        const int B = x.size(0), n = x.size(1), C = x.size(2);
        c10::DeviceGuard guard(x.device());
        Tensor w, f;
        if (w_in.has_value() && w_in->defined()) w = act(is_act_dtype(*w_in) ? *w_in : w_in->to(at::kFloat));
        if (f_in.has_value() && f_in->defined()) f = act(f_in->to(x.scalar_type()));
        const Tensor hp = f32c(H_pre), ho = f32c(H_post), hr = f32c(H_res);
        TORCH_CHECK(hp.numel() == n && ho.numel() == n && hr.numel() == n * n, "mhc: H shapes do not match n = ", n);
        Tensor y = at::empty({B, n, C}, x.options().dtype(out_dtype.value_or(at::kFloat)));
        Tensor small = at::empty({2 * n + n * n + B}, x.options().dtype(at::kFloat));  // Hpre | Hpost | M | q
        float *s = small.data_ptr<float>();
        Tensor ws = workspace(x, mhc_layer_static_workspace_bytes(B, n, C));
        check("mhc_layer_fwd",
              mhc_layer_fwd(ptr(x), dt(x), ptr(w), w.defined() ? dt(w) : 0, hp.data_ptr<float>(), ho.data_ptr<float>(),
                            hr.data_ptr<float>(), ptr(f), ptr(y), dt(y), s, s + n, s + 2 * n, s + 2 * n + n * n, B, n, C,
                            (int)iters, (float)eps, ws.data_ptr(), (size_t)ws.numel(), stream_of(x)));
        ctx->save_for_backward({x, w, hp, ho, hr, f, small});
        ctx->saved_data["iters"] = iters;
        ctx->saved_data["eps"] = eps;
        ctx->saved_data["x_dtype"] = (int64_t)x_in.scalar_type();
        ctx->saved_data["w_dtype"] = (int64_t)(w.defined() ? w_in->scalar_type() : at::kFloat);
        ctx->saved_data["f_dtype"] = (int64_t)(f.defined() ? f_in->scalar_type() : at::kFloat);
        ctx->saved_data["h_dtypes"] = std::vector<int64_t>{(int64_t)H_pre.scalar_type(), (int64_t)H_post.scalar_type(),
                                                           (int64_t)H_res.scalar_type()};
        ctx->saved_data["h_res_shape"] = H_res.sizes().vec();
        return y;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &x = saved[0], &w = saved[1], &hp = saved[2], &ho = saved[3], &hr = saved[4], &f = saved[5],
                     &small = saved[6];
        const int B = x.size(0), n = x.size(1), C = x.size(2);
        c10::DeviceGuard guard(x.device());
        // bfloat16 activations with a float32 result hand back a float32 gradient: it is rounded to the
        // activations' format here, so that the backward runs the kernels that take both in 2 bytes (the
        // mixed pair goes through slower general kernels: 111 against 20 us for dx at B=128 n=32 C=1280).
        // One pass also when the gradient arrives as a broadcast view (the backward of a sum).
        const bool round_dy = x.scalar_type() == at::kBFloat16 && grads[0].scalar_type() == at::kFloat;
        Tensor dy = act(round_dy ? grads[0].to(grads[0].options().dtype(at::kBFloat16), false, false, at::MemoryFormat::Contiguous)
                                 : grads[0]);
        const auto fo = x.options().dtype(at::kFloat);
        Tensor dx = at::empty_like(x);
        Tensor df = f.defined() ? at::empty_like(f) : Tensor();
        Tensor dw = f.defined() ? Tensor() : at::empty({C}, fo);
        Tensor dh = at::empty({2 * n + n * n}, fo);
        float *s = small.data_ptr<float>(), *d = dh.data_ptr<float>();
        Tensor ws = workspace(x, mhc_layer_static_workspace_bytes(B, n, C));
        check("mhc_layer_bwd",
              mhc_layer_bwd(ptr(dy), dt(dy), ptr(x), dt(x), ptr(w), w.defined() ? dt(w) : 0, hp.data_ptr<float>(),
                            ho.data_ptr<float>(), hr.data_ptr<float>(), ptr(f), s, s + n, s + 2 * n, s + 2 * n + n * n,
                            ptr(dx), ptr(df), dw.defined() ? dw.data_ptr<float>() : nullptr, d, d + n, d + 2 * n, B, n, C,
                            (int)ctx->saved_data["iters"].toInt(), (float)ctx->saved_data["eps"].toDouble(), ws.data_ptr(),
                            (size_t)ws.numel(), stream_of(x)));
        auto to = [](const Tensor &t, int64_t st) {
            const auto sc = (at::ScalarType)st;
            return t.scalar_type() == sc ? t : t.to(sc);
        };
        const auto hd = ctx->saved_data["h_dtypes"].toIntVector();
        variable_list out(9);
        out[0] = to(dx, ctx->saved_data["x_dtype"].toInt());
        out[1] = (dw.defined() && w.defined()) ? to(dw, ctx->saved_data["w_dtype"].toInt()) : Tensor();
        out[2] = to(dh.narrow(0, 0, n), hd[0]);
        out[3] = to(dh.narrow(0, n, n), hd[1]);
        out[4] = to(dh.narrow(0, 2 * n, n * n).reshape(ctx->saved_data["h_res_shape"].toIntVector()), hd[2]);
        out[8] = df.defined() ? to(df, ctx->saved_data["f_dtype"].toInt()) : Tensor();
        return out;
    }
};

// forward only: nothing is kept for a backward pass (coefficients stay in the workspace)
Tensor mhc_layer_inference(const Tensor &x_in, const Tensor &w_in, const Tensor &H_pre, const Tensor &H_post,
                           const Tensor &H_res, int64_t iters, double eps, c10::optional<at::ScalarType> out_dtype) {
    const Tensor x = act(is_act_dtype(x_in) ? x_in : x_in.to(at::kFloat));
    const Tensor w = act(is_act_dtype(w_in) ? w_in : w_in.to(at::kFloat));
    const int B = x.size(0), n = x.size(1), C = x.size(2);
    c10::DeviceGuard guard(x.device());
    const Tensor hp = f32c(H_pre), ho = f32c(H_post), hr = f32c(H_res);
    Tensor y = at::empty({B, n, C}, x.options().dtype(out_dtype.value_or(at::kFloat)));
    Tensor ws = workspace(x, mhc_layer_static_workspace_bytes(B, n, C));
    check("mhc_layer_fwd",
          mhc_layer_fwd(ptr(x), dt(x), ptr(w), dt(w), hp.data_ptr<float>(), ho.data_ptr<float>(), hr.data_ptr<float>(),
                        nullptr, ptr(y), dt(y), nullptr, nullptr, nullptr, nullptr, B, n, C, (int)iters, (float)eps,
                        ws.data_ptr(), (size_t)ws.numel(), stream_of(x)));
    return y;
}

// ---------------------------------------------------------------------------------------------
// stand-alone operators (reference ops.py:13-52, bindings.cu:115-164)
// ---------------------------------------------------------------------------------------------
struct SinkhornFn : public torch::autograd::Function<SinkhornFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &inp_in, int64_t iters, double eps) {
        const Tensor inp = f32c(inp_in);
        TORCH_CHECK(inp.dim() >= 2, "mhc: sinkhorn_knopp takes [..., rows, cols]");
        c10::DeviceGuard guard(inp.device());
        const int rows = inp.size(-2), cols = inp.size(-1);
        const int batch = (int)(inp.numel() / ((int64_t)rows * cols));
        Tensor out = at::empty_like(inp);
        check("mhc_sinkhorn_knopp_fwd", mhc_sinkhorn_knopp_fwd(inp.data_ptr<float>(), out.data_ptr<float>(), batch, rows,
                                                                cols, (int)iters, (float)eps, stream_of(inp)));
        ctx->save_for_backward({inp});
        ctx->saved_data["iters"] = iters;
        ctx->saved_data["eps"] = eps;
        ctx->saved_data["dtype"] = (int64_t)inp_in.scalar_type();
        return out;
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const Tensor inp = ctx->get_saved_variables()[0];
        c10::DeviceGuard guard(inp.device());
        const Tensor go = f32c(grads[0]);
        const int rows = inp.size(-2), cols = inp.size(-1);
        const int batch = (int)(inp.numel() / ((int64_t)rows * cols));
        const int iters = (int)ctx->saved_data["iters"].toInt();
        Tensor d_inp = at::empty_like(inp);
        Tensor ws = workspace(inp, mhc_sinkhorn_knopp_bwd_workspace_bytes(batch, rows, cols, iters));
        check("mhc_sinkhorn_knopp_bwd",
              mhc_sinkhorn_knopp_bwd(go.data_ptr<float>(), inp.data_ptr<float>(), d_inp.data_ptr<float>(), batch, rows, cols,
                                     iters, (float)ctx->saved_data["eps"].toDouble(), ws.data_ptr(), (size_t)ws.numel(),
                                     stream_of(inp)));
        const auto sd = (at::ScalarType)ctx->saved_data["dtype"].toInt();
        return {d_inp.scalar_type() == sd ? d_inp : d_inp.to(sd), Tensor(), Tensor()};
    }
};

struct RMSNormFn : public torch::autograd::Function<RMSNormFn> {
    static Tensor forward(AutogradContext *ctx, const Tensor &inp_in, const Tensor &w_in, double eps) {
        TORCH_CHECK(is_act_dtype(inp_in) && is_act_dtype(w_in), "mhc: rmsnorm takes float32 or bfloat16 tensors");
        const Tensor inp = act(inp_in), w = act(w_in);
        c10::DeviceGuard guard(inp.device());
        const int C = inp.size(-1);
        const int rows = (int)(inp.numel() / C);
        Tensor out = at::empty_like(inp);
        Tensor rms = at::empty({rows}, inp.options().dtype(at::kFloat));
        check("mhc_rmsnorm_fwd", mhc_rmsnorm_fwd(ptr(inp), dt(inp), ptr(w), dt(w), ptr(out), rms.data_ptr<float>(), rows, C,
                                                  (float)eps, stream_of(inp)));
        ctx->save_for_backward({inp, w, rms});
        return out;
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor &inp = saved[0], &w = saved[1], &rms = saved[2];
        c10::DeviceGuard guard(inp.device());
        const Tensor go = act(grads[0].scalar_type() == inp.scalar_type() ? grads[0] : grads[0].to(inp.scalar_type()));
        const int C = inp.size(-1);
        const int rows = (int)(inp.numel() / C);
        Tensor d_inp = at::empty_like(inp);
        Tensor d_w = at::empty({C}, inp.options().dtype(at::kFloat));
        Tensor ws = workspace(inp, mhc_rmsnorm_bwd_workspace_bytes(rows, C));
        check("mhc_rmsnorm_bwd",
              mhc_rmsnorm_bwd(ptr(go), ptr(inp), dt(inp), ptr(w), dt(w), rms.data_ptr<float>(), ptr(d_inp),
                              d_w.data_ptr<float>(), rows, C, ws.data_ptr(), (size_t)ws.numel(), stream_of(inp)));
        return {d_inp, d_w.scalar_type() == w.scalar_type() ? d_w : d_w.to(w.scalar_type()), Tensor()};
    }
};

py::object g_error_class;  // mhc._lib.MHCError, handed over at import

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "PyTorch-ROCm binding of libmhc_hip.so (C ABI: include/mhc_hip.h)";
    py::register_exception_translator([](std::exception_ptr p) {
        try {
            if (p) std::rethrow_exception(p);
        } catch (const MhcError &e) {
            if (g_error_class) {
                py::object exc = g_error_class(e.fn, e.status);
                PyErr_SetObject(g_error_class.ptr(), exc.ptr());
            } else {
                PyErr_SetString(PyExc_RuntimeError, e.what());
            }
        }
    });
    m.def("set_error_class", [](py::object cls) { g_error_class = std::move(cls); });
    m.def("set_param_cache", [](bool on) { g_param_cache = on; },
          "Opt in to reusing the packed phi / bias / alpha of a layer while the parameters' storage addresses and "
          "in-place version counters are unchanged.  Writes through `.data` do not bump the counters: leave it off "
          "(the default) if parameters are ever updated that way.");
    m.def("abi_version", []() { return mhc_abi_version(); });
    m.def("mhc_layer_dynamic",
          [](const Tensor &x, const OptTensor &w, const Tensor &phi_pre, const Tensor &phi_post, const Tensor &phi_res,
             const Tensor &alpha_pre, const Tensor &alpha_post, const Tensor &alpha_res, const Tensor &b_pre,
             const Tensor &b_post, const Tensor &b_res, int64_t iters, double eps, c10::optional<at::ScalarType> out_dtype,
             const OptTensor &f_inject, bool compute_bf16) {
              return MHCDynamicFn::apply(x, w, phi_pre, phi_post, phi_res, alpha_pre, alpha_post, alpha_res, b_pre, b_post,
                                         b_res, iters, eps, out_dtype, f_inject, at::GradMode::is_enabled(), compute_bf16);
          },
          py::arg("x"), py::arg("w"), py::arg("phi_pre"), py::arg("phi_post"), py::arg("phi_res"), py::arg("alpha_pre"),
          py::arg("alpha_post"), py::arg("alpha_res"), py::arg("b_pre"), py::arg("b_post"), py::arg("b_res"), py::arg("iters"),
          py::arg("eps"), py::arg("out_dtype"), py::arg("f_inject"), py::arg("compute_bf16") = false,
          "mhc_layer_fwd_dynamic / mhc_layer_bwd_dynamic with autograd (reference bindings.cu:405-542)");
    m.def("mhc_layer_static",
          [](const Tensor &x, const OptTensor &w, const Tensor &H_pre, const Tensor &H_post, const Tensor &H_res,
             int64_t iters, double eps, c10::optional<at::ScalarType> out_dtype, const OptTensor &f_inject) {
              return MHCStaticFn::apply(x, w, H_pre, H_post, H_res, iters, eps, out_dtype, f_inject);
          },
          "mhc_layer_fwd / mhc_layer_bwd with autograd (reference bindings.cu:264-401)");
    m.def("mhc_layer_inference", &mhc_layer_inference, "mhc_layer_fwd_inference (reference bindings.cu:221-262)");
    m.def("sinkhorn_knopp", [](const Tensor &inp, int64_t iters, double eps) { return SinkhornFn::apply(inp, iters, eps); });
    m.def("rmsnorm", [](const Tensor &inp, const Tensor &w, double eps) { return RMSNormFn::apply(inp, w, eps); });
}
