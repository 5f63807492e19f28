// Thin libtorch binding of libs2attn.so: registers the attention operators under the reference's own names and schemas
//   attention_kernels::forward, backward, permute_to_nhwc, permute_to_nchw      (attention_interface.cpp:85-119)
// for the CUDA dispatch key (ROCm tensors dispatch there), plus the two entry points that hand the forward's output and
// softmax normaliser to the backward (s2attn_kernels::forward_lse, backward_saved; the reference recomputes both,
// attention_cuda_bwd.cu:856-956).  Everything here is host code: argument checks (the conditions of attention_cuda_fwd.cu:
// 553-570 and attention_cuda_bwd.cu:874-893), output allocation, the plan cache, and one call into the C ABI on torch's
// current stream.  There is no CPU implementation: CPU tensors are refused with a clear error.
//
// Built by the Makefile next to it into torch_harmonics_amd/_C.so and loaded with torch.ops.load_library; the fake (meta)
// kernels and the autograd rules are registered from Python (torch_harmonics_amd/ops.py), as the reference does.

#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <list>
#include <mutex>
#include <utility>
#include <tuple>
#include <vector>

#include "../../include/s2attn.h"

namespace {

using at::Tensor;

void check_rc(int64_t rc, const char *what)
{
    if (rc < 0) {
        const char *msg = s2attn_last_error();
        TORCH_CHECK(false, what, ": ", (msg && *msg) ? msg : "error");
    }
}

int dtype_code(at::ScalarType t)
{
    switch (t) {
    case at::kFloat: return S2ATTN_F32;
    case at::kBFloat16: return S2ATTN_BF16;
    case at::kHalf: return S2ATTN_F16;
    default: TORCH_CHECK(false, "unsupported dtype ", t); return -1;
    }
}

void require_gpu(const Tensor &t, const char *name, const c10::Device &dev)
{
    TORCH_CHECK(t.is_cuda(), name, " is on ", t.device(), "; the s2attn operators only run on a ROCm GPU (no CPU implementation is shipped)");
    TORCH_CHECK(t.device() == dev, name, " is on ", t.device(), " but the other operands are on ", dev);
}

// Activations are contiguous NHWC (the reference's contract) or a COLUMN BLOCK of a contiguous row-major buffer: unit
// channel stride, one point stride ld >= channels for the longitude axis, latitude and batch strides that follow from it.
// That is what a slice buf[..., c0:c1] of a fused q | k | v projection is; the library reads it in place.
// Returns 0 for a packed tensor, else ld; raises for anything else.
int64_t point_stride(const Tensor &t, const char *name)
{
    if (t.is_contiguous()) return 0;
    const int64_t ld = t.stride(2);
    const bool ok = t.stride(3) == 1 && ld >= t.size(3) && ld % 4 == 0 && t.stride(1) == t.size(2) * ld && t.stride(0) == t.size(1) * t.size(2) * ld
                    && t.storage_offset() % 4 == 0;
    TORCH_CHECK(ok, name, " must be contiguous, or a column block of a contiguous (B, nlat, nlon, width) buffer with width and offset multiples of 4");
    return ld;
}

// Same conditions the reference entry points enforce (attention_cuda_fwd.cu:553-570, attention_cuda_bwd.cu:874-893).
void validate(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor *dy, const Tensor &quad_weights, const Tensor &col_idx,
              const Tensor &row_off, int64_t num_heads, int64_t nlon_in, int64_t nlat_out, int64_t nlon_out)
{
    TORCH_CHECK(nlon_in > 0 && nlon_out > 0 && (nlon_in % nlon_out == 0 || nlon_out % nlon_in == 0), "either nlon_in (", nlon_in,
                ") must be an integer multiple of nlon_out (", nlon_out, "), or vice versa");
    TORCH_CHECK(num_heads >= 1, "num_heads must be positive, got ", num_heads);
    const Tensor *ts[] = {&kx, &vx, &qy, dy};
    const char *names[] = {"kx", "vx", "qy", "dy"};
    for (int i = 0; i < 4; i++) {
        if (!ts[i]) continue;
        TORCH_CHECK(ts[i]->dim() == 4, names[i], " must be a 4-dimensional (B, nlat, nlon, heads*channels) tensor, got ", ts[i]->dim(), " dimensions");
        (void)point_stride(*ts[i], names[i]);
    }
    TORCH_CHECK(qy.size(3) % num_heads == 0, "q/k channel count (", qy.size(3), ") must be divisible by num_heads (", num_heads, ")");
    TORCH_CHECK(vx.size(3) % num_heads == 0, "v channel count (", vx.size(3), ") must be divisible by num_heads (", num_heads, ")");
    TORCH_CHECK(kx.scalar_type() == qy.scalar_type(), "k dtype (", kx.scalar_type(), ") must match q dtype (", qy.scalar_type(), ")");
    TORCH_CHECK(vx.scalar_type() == qy.scalar_type(), "v dtype (", vx.scalar_type(), ") must match q dtype (", qy.scalar_type(), ")");
    if (dy) TORCH_CHECK(dy->scalar_type() == qy.scalar_type(), "dy dtype (", dy->scalar_type(), ") must match q dtype (", qy.scalar_type(), ")");
    TORCH_CHECK(kx.size(3) == qy.size(3), "k and q must have the same channel count, got ", kx.size(3), " and ", qy.size(3));
    TORCH_CHECK(kx.size(0) == vx.size(0) && kx.size(1) == vx.size(1) && kx.size(2) == vx.size(2) && kx.size(0) == qy.size(0),
                "k and v must share (B, nlat_in, nlon_in) and q must share B");
    TORCH_CHECK(kx.size(2) == nlon_in && qy.size(1) == nlat_out && qy.size(2) == nlon_out, "tensor extents do not match nlon_in=", nlon_in,
                ", nlat_out=", nlat_out, ", nlon_out=", nlon_out);
    if (dy)
        TORCH_CHECK(dy->size(0) == qy.size(0) && dy->size(1) == qy.size(1) && dy->size(2) == qy.size(2) && dy->size(3) == vx.size(3),
                    "dy must have the shape of the forward output");
    TORCH_CHECK(quad_weights.numel() == kx.size(1), "quad_weights must have nlat_in = ", kx.size(1), " entries, got ", quad_weights.numel());
    TORCH_CHECK(col_idx.scalar_type() == at::kLong && row_off.scalar_type() == at::kLong, "col_idx and row_off must be int64");
    const auto t = qy.scalar_type();
    TORCH_CHECK(t == at::kFloat || t == at::kBFloat16 || t == at::kHalf || t == at::kDouble, "unsupported dtype ", t);
    const auto dev = kx.device();
    require_gpu(kx, "kx", dev), require_gpu(vx, "vx", dev), require_gpu(qy, "qy", dev);
    if (dy) require_gpu(*dy, "dy", dev);
    require_gpu(quad_weights, "quad_weights", dev), require_gpu(col_idx, "col_idx", dev), require_gpu(row_off, "row_off", dev);
}

// ---- plans ------------------------------------------------------------------------------------------------------------
// The reference re-sorts the CSR rows on the device in every call (attention_cuda_utils.cu:74-113).  Here psi is turned into
// the library's run-length plan once, on the host, the first time a (col_idx, row_off) pair is seen (one device-to-host
// copy), and the device copy of the plan is kept.  An entry holds its index tensors, so their addresses cannot be recycled
// for another psi while it lives, and an in-place edit of either bumps its version counter and misses the cache.  A caller
// that built the plan ahead of time (the module does, in its constructor) passes it in and nothing is copied at all.
struct PlanEntry {
    const void *col = nullptr, *row = nullptr, *blob_ptr = nullptr;
    int64_t ncol = 0, nrow = 0;
    uint32_t vcol = 0, vrow = 0, vblob = 0;
    c10::Device device = c10::Device(c10::kCPU);
    int64_t ext[4] = {0, 0, 0, 0};
    Tensor blob, keep_col, keep_row;
    s2attn_plan plan = {};
};

std::mutex g_plan_mutex;
std::list<PlanEntry> g_plans; // most recently used first
constexpr size_t MAX_PLANS = 32;

uint32_t version_of(const Tensor &t) { return t.is_inference() ? 0u : t._version(); }

s2attn_plan plan_for(const Tensor &col_idx, const Tensor &row_off, int64_t nlat_in, int64_t nlon_in, int64_t nlat_out, int64_t nlon_out,
                     const c10::optional<Tensor> &blob, const c10::OptionalArrayRef<int64_t> &header)
{
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    const bool given = blob.has_value() && blob->defined() && header.has_value();
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it) {
        const bool hit = given ? (it->blob_ptr == blob->data_ptr() && it->vblob == version_of(*blob) && it->device == blob->device())
                               : (it->blob_ptr == nullptr && it->col == col_idx.data_ptr() && it->row == row_off.data_ptr() && it->ncol == col_idx.numel()
                                  && it->nrow == row_off.numel() && it->vcol == version_of(col_idx) && it->vrow == version_of(row_off)
                                  && it->device == col_idx.device());
        if (hit && it->ext[0] == nlat_in && it->ext[1] == nlon_in && it->ext[2] == nlat_out && it->ext[3] == nlon_out) {
            g_plans.splice(g_plans.begin(), g_plans, it);
            return g_plans.front().plan;
        }
    }
    PlanEntry e;
    e.ext[0] = nlat_in, e.ext[1] = nlon_in, e.ext[2] = nlat_out, e.ext[3] = nlon_out;
    if (given) {
        TORCH_CHECK(blob->scalar_type() == at::kInt && blob->is_contiguous() && (int64_t)header->size() == S2ATTN_PLAN_HEADER_INTS
                        && (*header)[S2ATTN_PH_MAGIC] == S2ATTN_PLAN_MAGIC && (*header)[S2ATTN_PH_TOTAL] == blob->numel(),
                    "plan header does not describe this plan tensor");
        TORCH_CHECK(blob->is_cuda() && blob->device() == col_idx.device(), "plan is on ", blob->device(), " but psi is on ", col_idx.device());
        e.blob = *blob;
        e.blob_ptr = blob->data_ptr();
        e.vblob = version_of(*blob);
        e.device = blob->device();
        for (int i = 0; i < S2ATTN_PLAN_HEADER_INTS; i++) e.plan.header[i] = (int32_t)(*header)[i];
    } else {
        const bool up = nlon_out % nlon_in == 0 && nlon_out != nlon_in;
        const int64_t want = (up ? nlat_in : nlat_out) + 1;
        TORCH_CHECK(row_off.numel() == want, "row_off must have ", up ? "nlat_in" : "nlat_out", " + 1 = ", want, " entries, got ", row_off.numel());
        const Tensor ci = col_idx.detach().to(at::kCPU).contiguous(), ro = row_off.detach().to(at::kCPU).contiguous();
        const int64_t n = s2attn_plan_size(ci.data_ptr<int64_t>(), ro.data_ptr<int64_t>(), ci.numel(), (int)nlat_in, (int)nlon_in, (int)nlat_out, (int)nlon_out);
        check_rc(n, "s2attn_plan_size");
        Tensor host = at::empty({n}, at::TensorOptions().dtype(at::kInt));
        check_rc(s2attn_plan_build(ci.data_ptr<int64_t>(), ro.data_ptr<int64_t>(), ci.numel(), (int)nlat_in, (int)nlon_in, (int)nlat_out, (int)nlon_out,
                                   host.data_ptr<int32_t>(), n),
                 "s2attn_plan_build");
        std::copy(host.data_ptr<int32_t>(), host.data_ptr<int32_t>() + S2ATTN_PLAN_HEADER_INTS, e.plan.header);
        e.blob = host.to(col_idx.device());
        e.col = col_idx.data_ptr(), e.row = row_off.data_ptr(), e.ncol = col_idx.numel(), e.nrow = row_off.numel();
        e.vcol = version_of(col_idx), e.vrow = version_of(row_off), e.device = col_idx.device();
        e.keep_col = col_idx, e.keep_row = row_off;
    }
    e.plan.data = e.blob.data_ptr<int32_t>();
    g_plans.push_front(std::move(e));
    while (g_plans.size() > MAX_PLANS) g_plans.pop_back();
    return g_plans.front().plan;
}

s2attn_shape shape_of(const Tensor &kx, const Tensor &vx, const Tensor &qy, int64_t num_heads)
{
    s2attn_shape sh = {};
    sh.ld_k = (int)point_stride(kx, "kx"), sh.ld_v = (int)point_stride(vx, "vx"), sh.ld_q = (int)point_stride(qy, "qy");
    sh.batch = (int)kx.size(0), sh.num_heads = (int)num_heads;
    sh.nlat_in = (int)kx.size(1), sh.nlon_in = (int)kx.size(2), sh.nlat_out = (int)qy.size(1), sh.nlon_out = (int)qy.size(2);
    sh.ck = (int)(kx.size(3) / num_heads), sh.cv = (int)(vx.size(3) / num_heads);
    sh.dtype = dtype_code(qy.scalar_type());
    return sh;
}

void *current_stream(const c10::Device &dev) { return static_cast<void *>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).stream()); }

// ---- forward ------------------------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor> forward_impl(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &quad_weights, const Tensor &col_idx,
                                        const Tensor &row_off, int64_t num_heads, int64_t nlon_in, int64_t nlat_out, int64_t nlon_out, bool with_lse,
                                        const c10::optional<Tensor> &plan_blob, const c10::OptionalArrayRef<int64_t> &plan_header)
{
    validate(kx, vx, qy, nullptr, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out);
    if (qy.scalar_type() == at::kDouble) { // stored as fp64, computed in fp32 like the reference (attention_cuda_utils.cuh:185-190)
        auto r = forward_impl(kx.to(at::kFloat), vx.to(at::kFloat), qy.to(at::kFloat), quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out,
                              nlon_out, with_lse, plan_blob, plan_header);
        return {std::get<0>(r).to(at::kDouble), std::get<1>(r)};
    }
    Tensor y = at::empty({kx.size(0), nlat_out, nlon_out, vx.size(3)}, kx.options());
    Tensor lse = with_lse ? at::empty({kx.size(0), num_heads, nlat_out, nlon_out}, kx.options().dtype(at::kFloat)) : at::empty({0}, kx.options().dtype(at::kFloat));
    if (y.numel() == 0) return {y, lse};
    const s2attn_plan plan = plan_for(col_idx, row_off, kx.size(1), nlon_in, nlat_out, nlon_out, plan_blob, plan_header);
    const s2attn_shape sh = shape_of(kx, vx, qy, num_heads);
    const Tensor qw = quad_weights.to(at::kFloat).contiguous();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(kx.device());
    check_rc(s2attn_forward_lse(kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), qw.data_ptr<float>(), y.data_ptr(), with_lse ? lse.data_ptr<float>() : nullptr,
                                &plan, &sh, current_stream(kx.device())),
             "s2attn_forward_lse");
    return {y, lse};
}

Tensor forward(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &quad_weights, const Tensor &col_idx, const Tensor &row_off,
               int64_t num_heads, int64_t nlon_in, int64_t nlat_out, int64_t nlon_out)
{
    return std::get<0>(forward_impl(kx, vx, qy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, false, c10::nullopt, c10::nullopt));
}

std::tuple<Tensor, Tensor> forward_lse(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &quad_weights, const Tensor &col_idx,
                                       const Tensor &row_off, int64_t num_heads, int64_t nlon_in, int64_t nlat_out, int64_t nlon_out,
                                       const c10::optional<Tensor> &plan, c10::OptionalArrayRef<int64_t> plan_header)
{
    return forward_impl(kx, vx, qy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, true, plan, plan_header);
}

// ---- backward -----------------------------------------------------------------------------------------------------------
std::tuple<Tensor, Tensor, Tensor> backward_impl(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &dy, const Tensor *y, const Tensor *lse,
                                                 const Tensor &quad_weights, const Tensor &col_idx, const Tensor &row_off, int64_t num_heads,
                                                 int64_t nlon_in, int64_t nlat_out, int64_t nlon_out, const c10::optional<Tensor> &plan_blob,
                                                 const c10::OptionalArrayRef<int64_t> &plan_header)
{
    validate(kx, vx, qy, &dy, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out);
    const bool saved = y != nullptr;
    if (saved) {
        require_gpu(*y, "y", kx.device()), require_gpu(*lse, "lse", kx.device());
        TORCH_CHECK(y->sizes() == dy.sizes() && y->scalar_type() == dy.scalar_type(), "y must be the forward output (shape and dtype of dy)");
        (void)point_stride(*y, "y");
        TORCH_CHECK(lse->dim() == 4 && lse->size(0) == kx.size(0) && lse->size(1) == num_heads && lse->size(2) == nlat_out && lse->size(3) == nlon_out
                        && lse->scalar_type() == at::kFloat && lse->is_contiguous(),
                    "lse must be the contiguous fp32 (B, num_heads, nlat_out, nlon_out) tensor returned by forward_lse");
    }
    if (qy.scalar_type() == at::kDouble) {
        const Tensor yf = saved ? y->to(at::kFloat) : Tensor();
        auto r = backward_impl(kx.to(at::kFloat), vx.to(at::kFloat), qy.to(at::kFloat), dy.to(at::kFloat), saved ? &yf : nullptr, lse, quad_weights, col_idx,
                               row_off, num_heads, nlon_in, nlat_out, nlon_out, plan_blob, plan_header);
        return {std::get<0>(r).to(at::kDouble), std::get<1>(r).to(at::kDouble), std::get<2>(r).to(at::kDouble)};
    }
    // Gradients mirror the layout of their tensors: k | v (| q) that are column blocks of ONE buffer get their gradients as the
    // same column blocks of ONE new buffer, so that the caller's input gradient is a single GEMM over it.
    Tensor dk, dv, dq;
    const int64_t ldk = point_stride(kx, "kx"), ldv = point_stride(vx, "vx"), ldq = point_stride(qy, "qy");
    // (the column ranges must lie inside one row of the buffer and be pairwise disjoint: k and v given as the same or overlapping
    // slices would otherwise have their gradients written to the same addresses)
    auto cols = [](const Tensor &t, int64_t ld) { return std::pair<int64_t, int64_t>(t.storage_offset() % ld, t.storage_offset() % ld + t.size(3)); };
    auto disjoint = [](std::pair<int64_t, int64_t> a, std::pair<int64_t, int64_t> b) { return a.second <= b.first || b.second <= a.first; };
    bool kv_fused = ldk > 0 && ldk == ldv && kx.storage().is_alias_of(vx.storage()) && kx.storage_offset() / ldk == vx.storage_offset() / ldk;
    if (kv_fused) kv_fused = cols(kx, ldk).second <= ldk && cols(vx, ldk).second <= ldk && disjoint(cols(kx, ldk), cols(vx, ldk));
    bool all_fused = kv_fused && ldq == ldk && qy.storage().is_alias_of(kx.storage()) && qy.sizes().slice(0, 3) == kx.sizes().slice(0, 3)
                     && qy.storage_offset() / ldk == kx.storage_offset() / ldk;
    if (all_fused) all_fused = cols(qy, ldk).second <= ldk && disjoint(cols(qy, ldk), cols(kx, ldk)) && disjoint(cols(qy, ldk), cols(vx, ldk));
    if (kv_fused) {
        Tensor buf = at::empty({kx.size(0), kx.size(1), kx.size(2), ldk}, kx.options());
        const int64_t used = kx.size(3) + vx.size(3) + (all_fused ? qy.size(3) : 0);
        if (used != ldk) buf.zero_(); // columns of the buffer that belong to none of the three
        dk = buf.narrow(3, kx.storage_offset() % ldk, kx.size(3));
        dv = buf.narrow(3, vx.storage_offset() % ldk, vx.size(3));
        dq = all_fused ? buf.narrow(3, qy.storage_offset() % ldk, qy.size(3)) : at::empty(qy.sizes(), qy.options());
    } else {
        dk = at::empty(kx.sizes(), kx.options()), dv = at::empty(vx.sizes(), vx.options()), dq = at::empty(qy.sizes(), qy.options());
    }
    if (qy.numel() == 0 || kx.numel() == 0) return {dk.zero_(), dv.zero_(), dq.zero_()};
    const s2attn_plan plan = plan_for(col_idx, row_off, kx.size(1), nlon_in, nlat_out, nlon_out, plan_blob, plan_header);
    s2attn_shape sh = shape_of(kx, vx, qy, num_heads);
    sh.ld_dy = (int)point_stride(dy, "dy"), sh.ld_y = saved ? (int)point_stride(*y, "y") : 0;
    sh.ld_dk = (int)point_stride(dk, "dk"), sh.ld_dv = (int)point_stride(dv, "dv"), sh.ld_dq = (int)point_stride(dq, "dq");
    // the backward that is handed y and lse needs the two statistics per point only; the other one also recomputes y and lse
    const int64_t nbytes = saved ? s2attn_backward_saved_workspace_bytes(&sh) : s2attn_backward_workspace_bytes(&sh);
    check_rc(nbytes, "s2attn_backward_workspace_bytes");
    Tensor ws = at::empty({(nbytes + 3) / 4}, kx.options().dtype(at::kFloat));
    const Tensor qw = quad_weights.to(at::kFloat).contiguous();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(kx.device());
    void *stream = current_stream(kx.device());
    if (saved)
        check_rc(s2attn_backward_saved(kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), y->data_ptr(), lse->data_ptr<float>(), qw.data_ptr<float>(),
                                       dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), ws.data_ptr(), &plan, &sh, stream),
                 "s2attn_backward_saved");
    else
        check_rc(s2attn_backward(kx.data_ptr(), vx.data_ptr(), qy.data_ptr(), dy.data_ptr(), qw.data_ptr<float>(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(),
                                 ws.data_ptr(), &plan, &sh, stream),
                 "s2attn_backward");
    return {dk, dv, dq};
}

std::tuple<Tensor, Tensor, Tensor> backward(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &dy, const Tensor &quad_weights,
                                            const Tensor &col_idx, const Tensor &row_off, int64_t num_heads, int64_t nlon_in, int64_t nlat_out,
                                            int64_t nlon_out)
{
    return backward_impl(kx, vx, qy, dy, nullptr, nullptr, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, c10::nullopt, c10::nullopt);
}

std::tuple<Tensor, Tensor, Tensor> backward_saved(const Tensor &kx, const Tensor &vx, const Tensor &qy, const Tensor &dy, const Tensor &y, const Tensor &lse,
                                                  const Tensor &quad_weights, const Tensor &col_idx, const Tensor &row_off, int64_t num_heads,
                                                  int64_t nlon_in, int64_t nlat_out, int64_t nlon_out, const c10::optional<Tensor> &plan,
                                                  c10::OptionalArrayRef<int64_t> plan_header)
{
    return backward_impl(kx, vx, qy, dy, &y, &lse, quad_weights, col_idx, row_off, num_heads, nlon_in, nlat_out, nlon_out, plan, plan_header);
}

// ---- layout ---------------------------------------------------------------------------------------------------------------
Tensor permute(const Tensor &x, bool to_nhwc)
{
    TORCH_CHECK(x.dim() == 4, "expected a 4-dimensional tensor, got ", x.dim(), " dimensions");
    TORCH_CHECK(x.is_contiguous(), "layout conversion expects a contiguous tensor");
    TORCH_CHECK(x.is_cuda(), "x is on ", x.device(), "; the s2attn operators only run on a ROCm GPU (no CPU implementation is shipped)");
    const int64_t d0 = x.size(0), d1 = x.size(1), d2 = x.size(2), d3 = x.size(3);
    Tensor out = to_nhwc ? at::empty({d0, d2, d3, d1}, x.options()) : at::empty({d0, d3, d1, d2}, x.options());
    if (x.numel() == 0) return out;
    const int es = (int)x.element_size();
    TORCH_CHECK(es == 2 || es == 4 || es == 8, "layout conversion supports 2-, 4- and 8-byte elements, got ", x.scalar_type());
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    void *stream = current_stream(x.device());
    check_rc(to_nhwc ? s2attn_permute_to_nhwc(x.data_ptr(), out.data_ptr(), d0, d1, d2, d3, es, stream)
                     : s2attn_permute_to_nchw(x.data_ptr(), out.data_ptr(), d0, d1, d2, d3, es, stream),
             "s2attn_permute");
    return out;
}
Tensor permute_to_nhwc(const Tensor &x) { return permute(x, true); }
Tensor permute_to_nchw(const Tensor &x) { return permute(x, false); }

} // namespace

// Schema strings as in the reference (attention_interface.cpp:85-86, 114-119).
TORCH_LIBRARY(attention_kernels, m)
{
    m.def("permute_to_nhwc(Tensor x) -> Tensor", {at::Tag::pt2_compliant_tag});
    m.def("permute_to_nchw(Tensor x) -> Tensor", {at::Tag::pt2_compliant_tag});
    m.def("forward(Tensor kx, Tensor vx, Tensor qy, Tensor quad_weights, Tensor col_idx, Tensor row_off, int "
          "num_heads, int nlon_in, int nlat_out, int nlon_out) -> Tensor",
          {at::Tag::pt2_compliant_tag});
    m.def("backward(Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor quad_weights, Tensor col_idx, Tensor "
          "row_off, int num_heads, int nlon_in, int nlat_out, int nlon_out) -> (Tensor, Tensor, Tensor)",
          {at::Tag::pt2_compliant_tag});
}

TORCH_LIBRARY_IMPL(attention_kernels, CUDA, m)
{
    m.impl("permute_to_nhwc", &permute_to_nhwc);
    m.impl("permute_to_nchw", &permute_to_nchw);
    m.impl("forward", &forward);
    m.impl("backward", &backward);
}

// CPU tensors reach the same entry points, whose device check fails with this package's own message ("only run on a ROCm
// GPU"): there is no CPU implementation, and the dispatcher's "could not run with arguments from the CPU backend" says less.
TORCH_LIBRARY_IMPL(attention_kernels, CPU, m)
{
    m.impl("permute_to_nhwc", &permute_to_nhwc);
    m.impl("permute_to_nchw", &permute_to_nchw);
    m.impl("forward", &forward);
    m.impl("backward", &backward);
}

// The same pair with the forward's output and normaliser handed to the backward, and an optional plan built ahead of time.
TORCH_LIBRARY(s2attn_kernels, m)
{
    m.def("forward_lse(Tensor kx, Tensor vx, Tensor qy, Tensor quad_weights, Tensor col_idx, Tensor row_off, int num_heads, int nlon_in, int "
          "nlat_out, int nlon_out, Tensor? plan=None, int[]? plan_header=None) -> (Tensor, Tensor)",
          {at::Tag::pt2_compliant_tag});
    m.def("backward_saved(Tensor kx, Tensor vx, Tensor qy, Tensor dy, Tensor y, Tensor lse, Tensor quad_weights, Tensor col_idx, Tensor row_off, int "
          "num_heads, int nlon_in, int nlat_out, int nlon_out, Tensor? plan=None, int[]? plan_header=None) -> (Tensor, Tensor, Tensor)",
          {at::Tag::pt2_compliant_tag});
}

TORCH_LIBRARY_IMPL(s2attn_kernels, CUDA, m)
{
    m.impl("forward_lse", &forward_lse);
    m.impl("backward_saved", &backward_saved);
}

TORCH_LIBRARY_IMPL(s2attn_kernels, CPU, m) // fails with the same message as above
{
    m.impl("forward_lse", &forward_lse);
    m.impl("backward_saved", &backward_saved);
}
