// torch op registration for the HSTU attention family under the reference's names and schemas:
//   mxrec::hstu_jagged.equal / .delta   (cust_op/framework/torch_plugin/torch_library/hstu/hstu_jagged.cpp:186-231)
//   mxrec::hstu_jagged_backward.equal / .delta and the autograd formula of hstu_jagged (hstu_jagged.cpp:69-138,202-356)
//   mxrec::hstu_paged                    (hstu_paged.cpp:73-95)
//   mxrec::hstu_dense, hstu_dense_backward and the autograd formula of hstu_dense (hstu_dense.cpp:13-248)
// plus two ops the reference has no counterpart for (fused bias tables, fp8 paged cache).
// The host logic mirrors hstu_deltaq_forward_impl_npu (hstu_jagged.cpp:22-67): same checks and
// messages, same defaults, output allocated here; the device work is one call into the C ABI of
// libhstu_hip.so on the current stream.  There is no CPU implementation: CPU tensors get the same
// argument checks and then a clear error.
#include <ATen/ATen.h>
#include <ATen/CPUGeneratorImpl.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <cmath>
#include <limits>
#include <mutex>

#include "hstu_hip.h"
#include "hstu_bias.h"
#include "hstu_layer.h"

namespace mxrec_hstu {

constexpr int64_t kMinSeqLen = 1;
constexpr int64_t kMaxSeqLen = 20480;

static void mask_check(int64_t mask_type, bool mask_defined) {
    TORCH_CHECK(0 <= mask_type && mask_type <= 3, "maskType expect in [0, 3], but value is ", mask_type);
    TORCH_CHECK(mask_type != 1, "maskType current not support triu now, pls use custom mask");
    TORCH_CHECK(!(mask_type == 3 && !mask_defined), "use custom mask must have valid mask tensor");
}

static void max_seq_len_check(int64_t n) {
    TORCH_CHECK(n >= kMinSeqLen && n <= kMaxSeqLen, "maxSeqLen expect in [1, 20480], but value is ", n);
}

// `fp8`: float8_e4m3fn is taken too (the forward of the jagged and dense ops: hstu_jagged.cpp:53-54, output in fp16)
static int32_t io_dtype(const at::Tensor& t, const char* what, bool fp8 = false) {
    switch (t.scalar_type()) {
        case at::kFloat: return HSTU_F32;
        case at::kHalf: return HSTU_F16;
        case at::kBFloat16: return HSTU_BF16;
        case at::kFloat8_e4m3fn:
            if (fp8) return HSTU_FP8_E4M3;
            [[fallthrough]];
        default: TORCH_CHECK(false, what, " dtype expect float32, float16 or bfloat16", fp8 ? " or float8_e4m3fn" : "", ", but get ", t.scalar_type());
    }
    return -1;
}
static at::ScalarType out_type_of(const at::Tensor& q) { return q.scalar_type() == at::kFloat8_e4m3fn ? at::kHalf : q.scalar_type(); }

static const void* ptr_or_null(const at::Tensor& t) { return t.defined() ? t.const_data_ptr() : nullptr; }

struct Holder {  // keeps converted temporaries alive until the launch is queued
    std::vector<at::Tensor> keep;
    at::Tensor index(const c10::optional<at::Tensor>& t, at::ScalarType st, int64_t expect_len, const char* name) {
        if (!t.has_value() || !t->defined()) return at::Tensor();
        TORCH_CHECK(t->dim() == 1, name, " should have 1 dimension, but get ", t->dim());
        if (expect_len >= 0)
            TORCH_CHECK(t->size(0) == expect_len, "The length of ", name, " expect ", expect_len, ", but get ", t->size(0));
        auto x = t->to(st).contiguous();
        keep.push_back(x);
        return x;
    }
    at::Tensor same(const at::Tensor& t) {
        auto x = t.contiguous();
        keep.push_back(x);
        return x;
    }
};

static void require_gpu(const at::Tensor& q, const char* op) {
    TORCH_CHECK(q.is_cuda(), "mxrec::", op, " has no CPU implementation: move the tensors to the MI355X (device 'cuda')");
}

static void run_abi(int (*ws_fn)(const hstu_fwd_params*, uint64_t*), int (*fn)(const hstu_fwd_params*, void*, uint64_t, void*),
                    const hstu_fwd_params& p, const at::Tensor& q, const char* op) {
    uint64_t ws_bytes = 0;
    int rc = ws_fn(&p, &ws_bytes);
    TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
    require_gpu(q, op);
    at::Tensor ws;
    if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(q.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    rc = fn(&p, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
}

// ---------------------------------------------------------------------------------------------
// The layers of one model call the jagged op on one batch geometry: same offset tensors, same shapes and
// attributes, other q/k/v.  The work list in the workspace depends on the geometry only, so the last workspace of every
// (device, stream) is kept together with what it was built from, and a call that matches passes
// HSTU_FLAG_REUSE_WORKSPACE instead of building the list again.  The entry holds references to the offset / count
// tensors themselves: their storage cannot be handed to another tensor while it is cached, and an in-place write
// shows in their version counters.  Calls on one stream are ordered, so sharing the workspace between them is safe.
// ---------------------------------------------------------------------------------------------
struct ListCacheEntry {
    at::Tensor ws;
    std::vector<at::Tensor> geo;            // seq_offset, seq_offset_k, num_context, num_target (undefined where absent)
    std::vector<uint32_t> versions;
    hstu_fwd_params shape;                  // the scalar fields of the call that built it (pointers zeroed)
    void* stream = nullptr;
    int device = -1;
    unsigned long long capture = 0;         // id of the stream capture the list was built in (0: built by an eager call)
};

static hstu_fwd_params scalar_fields(hstu_fwd_params p) {
    p.q = p.k = p.v = nullptr; p.out = nullptr; p.mask = p.attn_bias = nullptr;
    p.seq_offset_q = p.seq_offset_k = p.num_context = p.num_target = nullptr;
    p.kv_cache = p.page_offsets = p.page_ids = p.last_page_len = nullptr; p.kv_scales = nullptr;
    p.pos_table = p.ts_table = p.ts_bounds = nullptr; p.timestamps = nullptr;
    p.silu_scale = 0.f; p.alpha = 0.f; p.flags = 0;
    return p;
}

// Id of the capture `stream` is recording into, 0 when it is not capturing.
static unsigned long long capture_id_of(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    if (hipStreamGetCaptureInfo(stream, &status, &id) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return status == hipStreamCaptureStatusActive ? (id ? id : ~0ull) : 0;
}

// A list is reused only where it is known to be current when the kernel runs:
//   * eager calls reuse the list of the last eager call on their (device, stream) -- the tensors' version counters show
//     in-place writes made through torch (writes that bypass them -- `.data`, a foreign kernel on the raw pointer -- do not);
//   * a call recorded into a stream capture reuses only a list that was built inside the same capture (its schedule
//     kernel then precedes it in the graph, so every replay rebuilds the list from the offsets of that replay), and its
//     workspace is allocated inside the capture, so it belongs to the graph's memory pool; eager calls never see it;
//   * tensors without a version counter (created under torch.inference_mode()) are not cached at all.
static void run_abi_cached(const hstu_fwd_params& p0, const at::Tensor& q, const std::vector<at::Tensor>& geo, const char* op) {
    static std::mutex mu;
    static std::vector<ListCacheEntry> cache;   // a handful of (device, stream) pairs, eager and capturing apart
    for (const auto& t : geo)
        if (t.defined() && t.is_inference()) {
            run_abi(hstu_hip_jagged_forward_get_workspace_size, hstu_hip_jagged_forward, p0, q, op);
            return;
        }
    hstu_fwd_params p = p0;
    uint64_t ws_bytes = 0;
    int rc = hstu_hip_jagged_forward_get_workspace_size(&p, &ws_bytes);
    TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
    require_gpu(q, op);
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(q.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    if (ws_bytes == 0) {
        rc = hstu_hip_jagged_forward(&p, nullptr, 0, (void*)stream.stream());
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        return;
    }
    const unsigned long long capture = capture_id_of(stream.stream());
    // what the list depends on besides the offsets: every scalar field, and which optional inputs are there
    hstu_fwd_params shape = scalar_fields(p);
    shape.flags = (p.attn_bias ? 1u : 0u) | (p.mask ? 2u : 0u) | (p.pos_table ? 4u : 0u) | (p.ts_table ? 8u : 0u);
    std::lock_guard<std::mutex> lock(mu);
    ListCacheEntry* hit = nullptr;
    ListCacheEntry* slot = nullptr;
    for (auto& e : cache)
        if (e.device == q.device().index() && e.stream == (void*)stream.stream() && (e.capture != 0) == (capture != 0)) slot = &e;
    if (slot && slot->capture == capture && slot->ws.defined() && (uint64_t)slot->ws.numel() >= ws_bytes &&
        std::memcmp(&slot->shape, &shape, sizeof(shape)) == 0) {
        bool same = true;
        for (size_t i = 0; i < geo.size(); i++) {
            const at::Tensor& a = slot->geo[i];
            same = same && a.defined() == geo[i].defined() &&
                   (!a.defined() || (a.is_same(geo[i]) && slot->versions[i] == geo[i]._version()));
        }
        if (same) hit = slot;
    }
    if (hit) {
        p.flags |= HSTU_FLAG_REUSE_WORKSPACE;
        rc = hstu_hip_jagged_forward(&p, hit->ws.data_ptr(), ws_bytes, (void*)stream.stream());
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        return;
    }
    if (!slot) {
        if (cache.size() >= 16) cache.erase(cache.begin());
        cache.emplace_back();
        slot = &cache.back();
    }
    // (a workspace of an earlier capture that is released here goes back to that graph's pool, which keeps it for the replays)
    slot->ws = at::empty({(int64_t)ws_bytes}, q.options().dtype(at::kByte));
    slot->geo = geo;
    slot->versions.clear();
    for (const auto& t : geo) slot->versions.push_back(t.defined() ? t._version() : 0u);
    slot->shape = shape;
    slot->stream = (void*)stream.stream();
    slot->device = q.device().index();
    slot->capture = capture;
    rc = hstu_hip_jagged_forward(&p, slot->ws.data_ptr(), ws_bytes, (void*)stream.stream());
    if (rc != HSTU_OK) slot->ws = at::Tensor();
    TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
}

// ---------------------------------------------------------------------------------------------
// Smallest fp32 |dt| of every time bucket, from the reference formula
//   bucket = trunc(log(clamp(|dt|, 1, e^(nb*div))) / div)   (cust_op/test/relative_attn_bias/torch/utils.py:115-123)
// evaluated with ATen's own CPU log so that the integer ids agree bit for bit with a torch evaluation
// of that formula.  bounds[0] = 0, bounds[nb+1] = +inf.
// ---------------------------------------------------------------------------------------------
static at::Tensor bucket_of(const at::Tensor& x, int64_t nb, double div) {
    float cmax = std::exp((float)(nb * div));
    return at::log(at::clamp(x, 1.0, (double)cmax)).div((float)div).to(at::kLong);
}

at::Tensor hstu_time_bucket_bounds(int64_t num_buckets, double bucket_divisor) {
    TORCH_CHECK(num_buckets >= 1 && num_buckets <= 4096, "num_buckets expect in [1, 4096], but value is ", num_buckets);
    TORCH_CHECK(bucket_divisor > 0, "bucket_divisor must be positive");
    const int64_t nb = num_buckets;
    auto opt_i = at::TensorOptions().dtype(at::kInt);
    // search over the bit patterns of positive floats (monotone as integers)
    float one = 1.0f, big = std::numeric_limits<float>::max();
    int32_t lo0, hi0;
    std::memcpy(&lo0, &one, 4);
    std::memcpy(&hi0, &big, 4);
    auto target = at::arange(1, nb + 1, at::kLong);
    auto lo = at::full({nb}, lo0, opt_i), hi = at::full({nb}, hi0, opt_i);
    auto reach = bucket_of(hi.view(at::kFloat), nb, bucket_divisor).ge(target);  // bucket attainable at all
    for (int it = 0; it < 34; ++it) {
        auto mid = lo + (hi - lo).div(2, "floor").to(at::kInt);
        auto ok = bucket_of(mid.view(at::kFloat), nb, bucket_divisor).ge(target);
        hi = at::where(ok, mid, hi);
        lo = at::where(ok, lo, at::minimum(mid + 1, hi));
    }
    auto b = hi.view(at::kFloat).clone();
    b = at::where(reach, b, at::full_like(b, std::numeric_limits<float>::infinity()));
    auto out = at::empty({nb + 2}, at::kFloat);
    out[0] = 0.0f;
    out.slice(0, 1, nb + 1).copy_(b);
    out[nb + 1] = std::numeric_limits<float>::infinity();
    return out;
}

static at::Tensor cached_bounds(int64_t nb, double div, const at::Device& dev) {
    static std::mutex mu;
    static std::vector<std::tuple<int64_t, double, at::Device, at::Tensor>> cache;
    std::lock_guard<std::mutex> g(mu);
    for (auto& e : cache)
        if (std::get<0>(e) == nb && std::get<1>(e) == div && std::get<2>(e) == dev) return std::get<3>(e);
    auto t = hstu_time_bucket_bounds(nb, div).to(dev);
    cache.emplace_back(nb, div, dev, t);
    return t;
}

// ---------------------------------------------------------------------------------------------
// jagged (equal / delta) + table-bias extension
// ---------------------------------------------------------------------------------------------
struct Tables {
    c10::optional<at::Tensor> pos_table, ts_table, timestamps;
    double bucket_divisor = 0.301;
};

static at::Tensor jagged_forward_impl(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                      const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                      int64_t mask_type, int64_t max_seq_len_q, int64_t max_seq_len_k, double silu_scale,
                                      const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                                      const c10::optional<at::Tensor>& num_context,
                                      const c10::optional<at::Tensor>& num_target,
                                      const c10::optional<int64_t>& target_group_size, const c10::optional<double>& alpha,
                                      bool deterministic, const Tables* tables, const char* op,
                                      const at::Tensor* grad = nullptr,
                                      std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor>* grads = nullptr) {
    TORCH_CHECK(q.dim() == 3, "The q should be 3D in jagged layout");
    TORCH_CHECK(k.dim() == 3 && v.dim() == 3, "The k and v should be 3D in jagged layout");
    TORCH_CHECK(seq_offset.defined() && seq_offset.dim() == 1 && seq_offset.size(0) >= 2,
                "acSeqOffset params error should have at least two element.");
    TORCH_CHECK(seq_offset_k.defined() && seq_offset_k.dim() == 1 && seq_offset_k.size(0) >= 2,
                "acSeqOffsetK params error should have at least two element.");
    TORCH_CHECK(seq_offset.scalar_type() == at::kInt || seq_offset.scalar_type() == at::kLong,
                "seq_offset dtype expect int32 or int64, but get ", seq_offset.scalar_type());
    TORCH_CHECK(seq_offset_k.size(0) == seq_offset.size(0), "seq_offset and seq_offset_k should have the same shape");
    Holder h;
    const auto it = seq_offset.scalar_type();
    const int64_t batch = seq_offset.size(0) - 1;
    auto off_q = h.same(seq_offset);
    auto off_k = h.index(seq_offset_k, it, -1, "seq_offset_k");
    auto dq = h.same(q), dk = h.same(k), dv = h.same(v);
    auto ctx = h.index(num_context, it, batch, "num_context");
    auto tgt = h.index(num_target, it, batch, "num_target");

    max_seq_len_check(max_seq_len_q);
    max_seq_len_check(max_seq_len_k);
    const bool mask_defined = mask.has_value() && mask->defined();
    mask_check(mask_type, mask_defined);

    const int32_t dt = io_dtype(dq, "q", grad == nullptr);
    TORCH_CHECK(dk.scalar_type() == dq.scalar_type() && dv.scalar_type() == dq.scalar_type(), "q, k, v dtype mismatch");
    TORCH_CHECK(dk.size(0) == dv.size(0), "K, V seqLens mismatch");
    TORCH_CHECK(dk.size(1) == dv.size(1), "K, V headNum mismatch");
    TORCH_CHECK(dq.size(2) == dk.size(2), "Q, K, V headDIM Shape Check failed");

    hstu_fwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.flags = deterministic ? HSTU_FLAG_DETERMINISTIC : 0u;
    p.dtype = dt;
    p.index_type = it == at::kLong ? HSTU_I64 : HSTU_I32;
    p.total_q = dq.size(0);
    p.total_k = dk.size(0);
    p.batch = (int32_t)batch;
    p.heads_q = (int32_t)dq.size(1);
    p.heads_k = (int32_t)dk.size(1);
    p.dim_qk = (int32_t)dq.size(2);
    p.dim_v = (int32_t)dv.size(2);
    p.mask_type = (int32_t)mask_type;
    p.max_seq_len_q = (int32_t)max_seq_len_q;
    p.max_seq_len_k = (int32_t)max_seq_len_k;
    p.target_group_size = (int32_t)target_group_size.value_or(0);
    p.silu_scale = (float)((silu_scale == 0.0) ? 1.0 / (double)max_seq_len_q : silu_scale);
    p.alpha = (float)alpha.value_or(1.0);

    at::Tensor dmask, dbias;
    const std::vector<int64_t> full = {batch, dq.size(1), max_seq_len_q, max_seq_len_k};
    if (mask_defined && mask_type == 3) {
        dmask = h.same(*mask);
        TORCH_CHECK(dmask.scalar_type() == dq.scalar_type(), "mask dtype must equal the q dtype");
        TORCH_CHECK(dmask.sizes() == at::IntArrayRef(full), "mask shape expect [batch, heads, max_seq_len, max_seq_len_k], but get ", dmask.sizes());
    }
    if (attn_bias.has_value() && attn_bias->defined()) {
        dbias = h.same(*attn_bias);
        TORCH_CHECK(dbias.scalar_type() == dq.scalar_type(), "attn_bias dtype must equal the q dtype");
        TORCH_CHECK(dbias.sizes() == at::IntArrayRef(full), "attn_bias shape expect [batch, heads, max_seq_len, max_seq_len_k], but get ", dbias.sizes());
    }
    at::Tensor pos, tst, tsb, tsv;
    if (tables) {
        if (tables->pos_table.has_value() && tables->pos_table->defined()) {
            pos = h.same(tables->pos_table->to(at::kFloat));
            TORCH_CHECK(pos.dim() == 1 && pos.size(0) == 2 * max_seq_len_k - 1, "pos_table expect 2*max_seq_len_k-1 = ",
                        2 * max_seq_len_k - 1, " entries, but get ", pos.sizes());
        }
        if (tables->ts_table.has_value() && tables->ts_table->defined()) {
            TORCH_CHECK(tables->timestamps.has_value() && tables->timestamps->defined(), "ts_table needs timestamps");
            tst = h.same(tables->ts_table->to(at::kFloat));
            tsv = h.same(tables->timestamps->to(at::kLong));
            TORCH_CHECK(tst.dim() == 1 && tst.size(0) >= 2, "ts_table expect num_buckets+1 entries");
            TORCH_CHECK(tsv.dim() == 1 && tsv.size(0) == dk.size(0), "timestamps expect one int64 per K row (", dk.size(0), "), but get ", tsv.sizes());
            tsb = cached_bounds(tst.size(0) - 1, tables->bucket_divisor, dq.device());
            p.num_buckets = (int32_t)(tst.size(0) - 1);
            p.ts_log2_scale = (float)(std::log(2.0) / tables->bucket_divisor);
        }
    }
    for (const at::Tensor* t : {&dk, &dv, &off_q, &off_k, &ctx, &tgt, &dmask, &dbias, &pos, &tst, &tsv})
        TORCH_CHECK(!t->defined() || t->device() == dq.device(), "all tensors must be on the device of q");

    at::Tensor out;
    if (!grad) out = at::empty({dq.size(0), dq.size(1), dv.size(2)}, dq.options().dtype(out_type_of(dq)));
    p.q = dq.const_data_ptr();
    p.k = dk.const_data_ptr();
    p.v = dv.const_data_ptr();
    p.out = grad ? nullptr : out.data_ptr();
    p.mask = ptr_or_null(dmask);
    p.attn_bias = ptr_or_null(dbias);
    p.seq_offset_q = off_q.const_data_ptr();
    p.seq_offset_k = off_k.const_data_ptr();
    p.num_context = ptr_or_null(ctx);
    p.num_target = ptr_or_null(tgt);
    p.pos_table = (const float*)ptr_or_null(pos);
    p.ts_table = (const float*)ptr_or_null(tst);
    p.ts_bounds = (const float*)ptr_or_null(tsb);
    p.timestamps = (const int64_t*)ptr_or_null(tsv);
    if (grad) {
        // the backward of the same call (reference: hstu_deltaq_backward_impl_npu, hstu_jagged.cpp:69-138): gradients
        // shaped like q, k, v, and like attn_bias when there is one (every element is written by the kernels)
        auto dgrad = h.same(*grad);
        TORCH_CHECK(dgrad.dim() == 3 && dgrad.size(0) == dq.size(0) && dgrad.size(1) == dq.size(1) && dgrad.size(2) == dv.size(2),
                    "grad shape expect [total_q, heads_q, dim_v], but get ", dgrad.sizes());
        TORCH_CHECK(dgrad.scalar_type() == dq.scalar_type() && dgrad.device() == dq.device(), "grad must have the dtype and device of q");
        hstu_bwd_params b;
        std::memset(&b, 0, sizeof(b));
        b.struct_size = sizeof(b);
        b.fwd = p;
        auto gq = at::empty_like(dq), gk = at::empty_like(dk), gv = at::empty_like(dv);
        at::Tensor gb;
        if (dbias.defined()) gb = at::empty_like(dbias);
        b.grad_out = dgrad.const_data_ptr();
        b.grad_q = gq.data_ptr();
        b.grad_k = gk.data_ptr();
        b.grad_v = gv.data_ptr();
        b.grad_bias = gb.defined() ? gb.data_ptr() : nullptr;
        uint64_t ws_bytes = 0;
        int rc = hstu_hip_jagged_backward_get_workspace_size(&b, &ws_bytes);
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        require_gpu(dq, op);
        at::Tensor ws;
        if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, dq.options().dtype(at::kByte));
        c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dq.device());
        auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
        rc = hstu_hip_jagged_backward(&b, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, (void*)stream.stream());
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        *grads = std::make_tuple(gq, gk, gv, gb);
        return at::Tensor();
    }
    // the tensors the caller handed in (not converted copies, which are new objects every call) identify the geometry
    auto opt = [](const c10::optional<at::Tensor>& t) { return t.has_value() ? *t : at::Tensor(); };
    const bool caller_owns = off_q.is_same(seq_offset) && off_k.is_same(seq_offset_k) &&
                             (!ctx.defined() || ctx.is_same(opt(num_context))) && (!tgt.defined() || tgt.is_same(opt(num_target)));
    if (caller_owns) run_abi_cached(p, dq, {off_q, off_k, ctx, tgt}, op);
    else run_abi(hstu_hip_jagged_forward_get_workspace_size, hstu_hip_jagged_forward, p, dq, op);
    return out;
}

at::Tensor hstu_jagged_equal(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                             const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                             int64_t mask_type, int64_t max_seq_len, double silu_scale, const at::Tensor& seq_offset,
                             const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                             c10::optional<int64_t> target_group_size, c10::optional<double> alpha, bool deterministic) {
    return jagged_forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len, silu_scale, seq_offset,
                               seq_offset, num_context, num_target, target_group_size, alpha, deterministic, nullptr,
                               "hstu_jagged");
}

at::Tensor hstu_jagged_delta(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                             const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                             int64_t mask_type, int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale,
                             const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                             const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                             c10::optional<int64_t> target_group_size, c10::optional<double> alpha, bool deterministic) {
    return jagged_forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset,
                               seq_offset_k, num_context, num_target, target_group_size, alpha, deterministic, nullptr,
                               "hstu_jagged");
}

using GradTuple = std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor>;

GradTuple hstu_jagged_backward_equal(const at::Tensor& grad, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                     const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                     int64_t mask_type, int64_t max_seq_len, double silu_scale, const at::Tensor& seq_offset,
                                     const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                                     c10::optional<int64_t> target_group_size, c10::optional<double> alpha) {
    GradTuple g;
    jagged_forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len, silu_scale, seq_offset, seq_offset,
                        num_context, num_target, target_group_size, alpha, false, nullptr, "hstu_jagged_backward", &grad, &g);
    return g;
}

GradTuple hstu_jagged_backward_delta(const at::Tensor& grad, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                     const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                     int64_t mask_type, int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale,
                                     const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                                     const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                                     c10::optional<int64_t> target_group_size, c10::optional<double> alpha) {
    GradTuple g;
    jagged_forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset, seq_offset_k,
                        num_context, num_target, target_group_size, alpha, false, nullptr, "hstu_jagged_backward", &grad, &g);
    return g;
}

// Autograd wiring of hstu_jagged.equal / .delta, as the reference's HstuJaggedNpuFusion (hstu_jagged.cpp:258-345): the
// forward saves its inputs, the backward calls the backward op and returns gradients for q, k, v and attn_bias.
class HstuJaggedFunction : public torch::autograd::Function<HstuJaggedFunction> {
public:
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                              const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias, int64_t mask_type,
                              int64_t max_seq_len_q, int64_t max_seq_len_k, double silu_scale, const at::Tensor& seq_offset_q,
                              const at::Tensor& seq_offset_k, const c10::optional<at::Tensor>& num_context,
                              const c10::optional<at::Tensor>& num_target, c10::optional<int64_t> target_group_size,
                              c10::optional<double> alpha, bool deterministic) {
        at::AutoDispatchBelowADInplaceOrView guard;
        ctx->save_for_backward({q, k, v, mask.value_or(at::Tensor()), attn_bias.value_or(at::Tensor()),
                                num_context.value_or(at::Tensor()), num_target.value_or(at::Tensor()), seq_offset_q, seq_offset_k});
        ctx->saved_data["mask_type"] = mask_type;
        ctx->saved_data["max_seq_len_q"] = max_seq_len_q;
        ctx->saved_data["max_seq_len_k"] = max_seq_len_k;
        ctx->saved_data["silu_scale"] = silu_scale;
        ctx->saved_data["target_group_size"] = target_group_size.value_or(0);
        ctx->saved_data["alpha"] = alpha.value_or(1.0);
        return jagged_forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset_q,
                                   seq_offset_k, num_context, num_target, target_group_size, alpha, deterministic, nullptr, "hstu_jagged");
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list grad_outputs) {
        const auto saved = ctx->get_saved_variables();
        auto opt = [](const at::Tensor& t) { return t.defined() ? c10::optional<at::Tensor>(t) : c10::nullopt; };
        GradTuple g;
        jagged_forward_impl(saved[0], saved[1], saved[2], opt(saved[3]), opt(saved[4]), ctx->saved_data["mask_type"].toInt(),
                            ctx->saved_data["max_seq_len_q"].toInt(), ctx->saved_data["max_seq_len_k"].toInt(),
                            ctx->saved_data["silu_scale"].toDouble(), saved[7], saved[8], opt(saved[5]), opt(saved[6]),
                            ctx->saved_data["target_group_size"].toInt(), ctx->saved_data["alpha"].toDouble(), false, nullptr,
                            "hstu_jagged_backward", &grad_outputs[0], &g);
        // one entry per forward argument: q, k, v, mask, attn_bias, then the eleven attributes and index tensors
        torch::autograd::tensor_list out(16);
        out[0] = std::get<0>(g);
        out[1] = std::get<1>(g);
        out[2] = std::get<2>(g);
        out[4] = std::get<3>(g);
        return out;
    }
};

at::Tensor hstu_jagged_equal_autograd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                      const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                      int64_t mask_type, int64_t max_seq_len, double silu_scale, const at::Tensor& seq_offset,
                                      const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                                      c10::optional<int64_t> target_group_size, c10::optional<double> alpha, bool deterministic) {
    return HstuJaggedFunction::apply(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len, silu_scale, seq_offset, seq_offset,
                                     num_context, num_target, target_group_size, alpha, deterministic);
}

at::Tensor hstu_jagged_delta_autograd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                      const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                      int64_t mask_type, int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale,
                                      const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                                      const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                                      c10::optional<int64_t> target_group_size, c10::optional<double> alpha, bool deterministic) {
    return HstuJaggedFunction::apply(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset, seq_offset_k,
                                     num_context, num_target, target_group_size, alpha, deterministic);
}

at::Tensor hstu_jagged_table_bias(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                  const c10::optional<at::Tensor>& pos_table, const c10::optional<at::Tensor>& ts_table,
                                  const c10::optional<at::Tensor>& timestamps, const c10::optional<at::Tensor>& attn_bias,
                                  int64_t mask_type, int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale,
                                  const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                                  const c10::optional<at::Tensor>& num_context, const c10::optional<at::Tensor>& num_target,
                                  c10::optional<int64_t> target_group_size, c10::optional<double> alpha,
                                  double bucket_divisor) {
    Tables t;
    t.pos_table = pos_table;
    t.ts_table = ts_table;
    t.timestamps = timestamps;
    t.bucket_divisor = bucket_divisor;
    return jagged_forward_impl(q, k, v, c10::nullopt, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale,
                               seq_offset, seq_offset_k, num_context, num_target, target_group_size, alpha, false, &t,
                               "hstu_jagged_table_bias");
}

// ---------------------------------------------------------------------------------------------
// paged (+ fp8 cache extension)
// ---------------------------------------------------------------------------------------------
static void check_non_empty(const at::Tensor& t, const char* name) {
    TORCH_CHECK(t.defined() && t.numel() > 0, name, " must be a non-empty tensor");
}

static at::Tensor paged_forward_impl(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                     const at::Tensor& kv_cache, const c10::optional<at::Tensor>& kv_scales,
                                     const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                                     int64_t mask_type, int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale,
                                     const at::Tensor& seq_offset, const at::Tensor& seq_offset_k,
                                     const at::Tensor& seq_offset_t, const at::Tensor& page_offsets,
                                     const at::Tensor& page_ids, const at::Tensor& last_page_len,
                                     const at::Tensor& num_target, int64_t target_group_size,
                                     const c10::optional<double>& alpha, bool deterministic, const char* op) {
    check_non_empty(kv_cache, "kv_cache");
    check_non_empty(page_ids, "page_ids");
    check_non_empty(last_page_len, "last_page_len");
    TORCH_CHECK(q.dim() == 3, "The q should be 3D in jagged layout");
    TORCH_CHECK(k.dim() == 3 && v.dim() == 3, "The k and v should be 3D in jagged layout");
    TORCH_CHECK(seq_offset.defined() && seq_offset.dim() == 1 && seq_offset.size(0) >= 2,
                "acSeqOffsetq params error should have at least two element.");
    TORCH_CHECK(seq_offset_k.defined() && seq_offset_k.dim() == 1 && seq_offset_k.size(0) >= 2,
                "acSeqOffsetK params error should have at least two element.");
    TORCH_CHECK(seq_offset_t.defined() && seq_offset_t.dim() == 1 && seq_offset_t.size(0) >= 2,
                "acSeqOffsetT params error should have at least two element.");
    TORCH_CHECK(seq_offset.scalar_type() == at::kInt || seq_offset.scalar_type() == at::kLong,
                "seq_offset dtype expect int32 or int64, but get ", seq_offset.scalar_type());
    TORCH_CHECK(seq_offset.size(0) == seq_offset_k.size(0) && seq_offset.size(0) == seq_offset_t.size(0),
                "offsetsLenQ, offsetsLenK and offsetsLenT should have the same shape.");
    Holder h;
    const auto it = seq_offset.scalar_type();
    const int64_t batch = seq_offset.size(0) - 1;
    auto off_q = h.same(seq_offset);
    auto off_k = h.index(seq_offset_k, it, -1, "seq_offset_k");
    auto poff = h.index(page_offsets, it, batch + 1, "page_offsets");
    auto pids = h.index(page_ids, it, -1, "page_ids");
    auto plast = h.index(last_page_len, it, batch, "last_page_len");
    auto dq = h.same(q), dk = h.same(k), dv = h.same(v), cache = h.same(kv_cache);

    max_seq_len_check(max_seq_len);
    max_seq_len_check(max_seq_len_k);
    const bool mask_defined = mask.has_value() && mask->defined();
    mask_check(mask_type, mask_defined);
    TORCH_CHECK(!num_target.defined() || target_group_size > 0,
                "targetGroupSize must be greater than 0 when numTarget is defined");
    auto tgt = h.index(num_target, it, batch, "num_target");

    const int32_t dt = io_dtype(dq, "q");
    TORCH_CHECK(dk.scalar_type() == dq.scalar_type() && dv.scalar_type() == dq.scalar_type(), "q, k, v dtype mismatch");
    TORCH_CHECK(dk.sizes() == dv.sizes(), "K, V shape mismatch");
    TORCH_CHECK(dq.size(2) == dk.size(2), "Q, K, V headDIM Shape Check failed");
    TORCH_CHECK(cache.dim() == 5 && cache.size(1) == 2, "kv_cache expect [pages, 2, page_size, heads, dim], but get ", cache.sizes());
    TORCH_CHECK(cache.size(3) == dk.size(1) && cache.size(4) == dk.size(2), "kv_cache heads/dim must match k");

    hstu_fwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.flags = deterministic ? HSTU_FLAG_DETERMINISTIC : 0u;
    p.dtype = dt;
    p.index_type = it == at::kLong ? HSTU_I64 : HSTU_I32;
    p.total_q = dq.size(0);
    p.total_k = dk.size(0);
    p.batch = (int32_t)batch;
    p.heads_q = (int32_t)dq.size(1);
    p.heads_k = (int32_t)dk.size(1);
    p.dim_qk = (int32_t)dq.size(2);
    p.dim_v = (int32_t)dv.size(2);
    p.mask_type = (int32_t)mask_type;
    p.max_seq_len_q = (int32_t)max_seq_len;
    p.max_seq_len_k = (int32_t)max_seq_len_k;
    p.target_group_size = (int32_t)target_group_size;
    p.silu_scale = (float)((silu_scale == 0.0) ? 1.0 / (double)max_seq_len : silu_scale);
    p.alpha = (float)alpha.value_or(1.0);
    p.num_pages = cache.size(0);
    p.page_size = (int32_t)cache.size(2);

    at::Tensor scales;
    const bool fp8 = cache.scalar_type() == at::kFloat8_e4m3fn || cache.scalar_type() == at::kByte;
    if (fp8) {
        TORCH_CHECK(kv_scales.has_value() && kv_scales->defined(), "fp8 kv_cache needs kv_scales [pages, 2, heads]");
        scales = h.same(kv_scales->to(at::kFloat));
        TORCH_CHECK(scales.dim() == 3 && scales.size(0) == cache.size(0) && scales.size(1) == 2 && scales.size(2) == cache.size(3),
                    "kv_scales expect [pages, 2, heads], but get ", scales.sizes());
        p.cache_dtype = HSTU_FP8_E4M3;
    } else {
        TORCH_CHECK(cache.scalar_type() == dq.scalar_type(), "kv_cache dtype must equal the q dtype (or be float8_e4m3fn with kv_scales)");
        p.cache_dtype = dt;
    }
    at::Tensor dmask, dbias;
    const std::vector<int64_t> full = {batch, dq.size(1), max_seq_len, max_seq_len_k};
    if (mask_defined && mask_type == 3) {
        dmask = h.same(*mask);
        TORCH_CHECK(dmask.scalar_type() == dq.scalar_type(), "mask dtype must equal the q dtype");
        TORCH_CHECK(dmask.sizes() == at::IntArrayRef(full), "mask shape expect [batch, heads, max_seq_len, max_seq_len_k], but get ", dmask.sizes());
    }
    if (attn_bias.has_value() && attn_bias->defined()) {
        dbias = h.same(*attn_bias);
        TORCH_CHECK(dbias.scalar_type() == dq.scalar_type(), "attn_bias dtype must equal the q dtype");
        TORCH_CHECK(dbias.sizes() == at::IntArrayRef(full), "attn_bias shape expect [batch, heads, max_seq_len, max_seq_len_k], but get ", dbias.sizes());
    }
    for (const at::Tensor* t : {&dk, &dv, &cache, &off_q, &off_k, &poff, &pids, &plast, &tgt, &dmask, &dbias, &scales})
        TORCH_CHECK(!t->defined() || t->device() == dq.device(), "all tensors must be on the device of q");

    auto out = at::empty_like(dq);
    p.q = dq.const_data_ptr();
    p.k = dk.const_data_ptr();
    p.v = dv.const_data_ptr();
    p.out = out.data_ptr();
    p.mask = ptr_or_null(dmask);
    p.attn_bias = ptr_or_null(dbias);
    p.seq_offset_q = off_q.const_data_ptr();
    p.seq_offset_k = off_k.const_data_ptr();
    p.num_target = ptr_or_null(tgt);
    p.kv_cache = cache.const_data_ptr();
    p.page_offsets = poff.const_data_ptr();
    p.page_ids = pids.const_data_ptr();
    p.last_page_len = plast.const_data_ptr();
    p.kv_scales = (const float*)ptr_or_null(scales);
    run_abi(hstu_hip_paged_forward_get_workspace_size, hstu_hip_paged_forward, p, dq, op);
    return out;
}

at::Tensor hstu_paged(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& kv_cache,
                      const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias, int64_t mask_type,
                      int64_t max_seq_len, int64_t max_seq_len_k, double silu_scale, const at::Tensor& seq_offset,
                      const at::Tensor& seq_offset_k, const at::Tensor& seq_offset_t, const at::Tensor& page_offsets,
                      const at::Tensor& page_ids, const at::Tensor& last_page_len, const at::Tensor& num_target,
                      int64_t target_group_size, c10::optional<double> alpha, bool deterministic) {
    return paged_forward_impl(q, k, v, kv_cache, c10::nullopt, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k,
                              silu_scale, seq_offset, seq_offset_k, seq_offset_t, page_offsets, page_ids, last_page_len,
                              num_target, target_group_size, alpha, deterministic, "hstu_paged");
}

at::Tensor hstu_paged_fp8(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& kv_cache,
                          const at::Tensor& kv_scales, const c10::optional<at::Tensor>& mask,
                          const c10::optional<at::Tensor>& attn_bias, int64_t mask_type, int64_t max_seq_len,
                          int64_t max_seq_len_k, double silu_scale, const at::Tensor& seq_offset,
                          const at::Tensor& seq_offset_k, const at::Tensor& seq_offset_t, const at::Tensor& page_offsets,
                          const at::Tensor& page_ids, const at::Tensor& last_page_len, const at::Tensor& num_target,
                          int64_t target_group_size, c10::optional<double> alpha, bool deterministic) {
    TORCH_CHECK(kv_cache.defined() && (kv_cache.scalar_type() == at::kFloat8_e4m3fn || kv_cache.scalar_type() == at::kByte),
                "hstu_paged_fp8 expects a float8_e4m3fn (or uint8 bit pattern) kv_cache");
    return paged_forward_impl(q, k, v, kv_cache, kv_scales, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k,
                              silu_scale, seq_offset, seq_offset_k, seq_offset_t, page_offsets, page_ids, last_page_len,
                              num_target, target_group_size, alpha, deterministic, "hstu_paged_fp8");
}

// ---------------------------------------------------------------------------------------------
// dense
// ---------------------------------------------------------------------------------------------
static at::Tensor dense_impl(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const c10::optional<at::Tensor>& mask,
                             const c10::optional<at::Tensor>& attn_bias, int64_t mask_type, int64_t max_seq_len, double silu_scale,
                             const char* op, const at::Tensor* grad = nullptr, GradTuple* grads = nullptr) {
    TORCH_CHECK(q.dim() == 4, "The q should be 4D in dense layout");
    Holder h;
    auto dq = h.same(q), dk = h.same(k), dv = h.same(v);
    max_seq_len_check(max_seq_len);
    const bool mask_defined = mask.has_value() && mask->defined();
    mask_check(mask_type, mask_defined);
    const int32_t dt = io_dtype(dq, "q", grad == nullptr);
    TORCH_CHECK(dk.scalar_type() == dq.scalar_type() && dv.scalar_type() == dq.scalar_type(), "q, k, v dtype mismatch");
    TORCH_CHECK(dq.sizes() == dk.sizes() && dq.sizes() == dv.sizes(), "dense layout needs q, k and v of one shape");
    TORCH_CHECK(dq.size(1) == max_seq_len, "dense layout: max_seq_len must equal the sequence dimension of q (", dq.size(1), ")");

    hstu_fwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = dt;
    p.index_type = HSTU_I64;
    p.batch = (int32_t)dq.size(0);
    p.total_q = p.total_k = dq.size(0) * dq.size(1);
    p.heads_q = p.heads_k = (int32_t)dq.size(2);
    p.dim_qk = p.dim_v = (int32_t)dq.size(3);
    p.mask_type = (int32_t)mask_type;
    p.max_seq_len_q = p.max_seq_len_k = (int32_t)max_seq_len;
    p.silu_scale = (float)((silu_scale == 0.0) ? 1.0 / (double)max_seq_len : silu_scale);
    p.alpha = 1.0f;
    at::Tensor dmask, dbias;
    const std::vector<int64_t> full = {dq.size(0), dq.size(2), max_seq_len, max_seq_len};
    if (mask_defined && mask_type == 3) {
        dmask = h.same(*mask);
        TORCH_CHECK(dmask.scalar_type() == dq.scalar_type(), "mask dtype must equal the q dtype");
        TORCH_CHECK(dmask.sizes() == at::IntArrayRef(full), "mask shape expect [batch, heads, seq, seq], but get ", dmask.sizes());
    }
    if (attn_bias.has_value() && attn_bias->defined()) {
        dbias = h.same(*attn_bias);
        TORCH_CHECK(dbias.scalar_type() == dq.scalar_type(), "attn_bias dtype must equal the q dtype");
        TORCH_CHECK(dbias.sizes() == at::IntArrayRef(full), "attn_bias shape expect [batch, heads, seq, seq], but get ", dbias.sizes());
    }
    p.q = dq.const_data_ptr();
    p.k = dk.const_data_ptr();
    p.v = dv.const_data_ptr();
    p.mask = ptr_or_null(dmask);
    p.attn_bias = ptr_or_null(dbias);
    if (grad) {
        // reference: hstu_dense_backward_impl_npu (hstu_dense.cpp:43-153).  Gradients shaped like q, k, v; the fourth
        // output is the bias gradient, or without a bias the reference's zero tensor with the sequence dimension
        // rounded up to a multiple of 256
        auto dgrad = h.same(*grad);
        TORCH_CHECK(dgrad.dim() == 4, "The grad should be 4D in normal layout");
        TORCH_CHECK(dgrad.sizes() == dq.sizes(), "Q and grad batch size check failed");
        TORCH_CHECK(dgrad.scalar_type() == dq.scalar_type() && dgrad.device() == dq.device(),
                    "grad dtype should be the same as q dtype, but got grad: ", dgrad.scalar_type(), " and q: ", dq.scalar_type());
        hstu_bwd_params b;
        std::memset(&b, 0, sizeof(b));
        b.struct_size = sizeof(b);
        b.fwd = p;
        auto gq = at::empty_like(dq), gk = at::empty_like(dk), gv = at::empty_like(dv);
        at::Tensor gb;
        if (dbias.defined()) gb = at::empty_like(dbias);
        b.grad_out = dgrad.const_data_ptr();
        b.grad_q = gq.data_ptr();
        b.grad_k = gk.data_ptr();
        b.grad_v = gv.data_ptr();
        b.grad_bias = gb.defined() ? gb.data_ptr() : nullptr;
        uint64_t ws_bytes = 0;
        int rc = hstu_hip_dense_backward_get_workspace_size(&b, &ws_bytes);
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        require_gpu(dq, op);
        at::Tensor ws;
        if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, dq.options().dtype(at::kByte));
        c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dq.device());
        auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
        rc = hstu_hip_dense_backward(&b, ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, (void*)stream.stream());
        TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
        if (!gb.defined()) {
            const int64_t padded = (max_seq_len + 255) / 256 * 256;
            gb = at::zeros({dq.size(0), dq.size(2), padded, padded}, dq.options());
        }
        *grads = std::make_tuple(gq, gk, gv, gb);
        return at::Tensor();
    }
    auto out = at::empty(dq.sizes(), dq.options().dtype(out_type_of(dq)));
    p.out = out.data_ptr();
    run_abi(hstu_hip_dense_forward_get_workspace_size, hstu_hip_dense_forward, p, dq, op);
    return out;
}

at::Tensor hstu_dense(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const c10::optional<at::Tensor>& mask,
                      const c10::optional<at::Tensor>& attn_bias, int64_t mask_type, int64_t max_seq_len, double silu_scale) {
    return dense_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale, "hstu_dense");
}

GradTuple hstu_dense_backward(const at::Tensor& grad, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                              const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                              int64_t mask_type, int64_t max_seq_len, double silu_scale) {
    GradTuple g;
    dense_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale, "hstu_dense_backward", &grad, &g);
    return g;
}

// Autograd wiring of hstu_dense, as the reference's HstuDenseNpuFusion (hstu_dense.cpp:177-235): gradients for q, k, v
// and, when given, attn_bias.
class HstuDenseFunction : public torch::autograd::Function<HstuDenseFunction> {
public:
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                              const c10::optional<at::Tensor>& mask, const c10::optional<at::Tensor>& attn_bias,
                              int64_t mask_type, int64_t max_seq_len, double silu_scale) {
        at::AutoDispatchBelowADInplaceOrView guard;
        ctx->save_for_backward({q, k, v, mask.value_or(at::Tensor()), attn_bias.value_or(at::Tensor())});
        ctx->saved_data["mask_type"] = mask_type;
        ctx->saved_data["max_seq_len"] = max_seq_len;
        ctx->saved_data["silu_scale"] = silu_scale;
        return hstu_dense(q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list grad_outputs) {
        auto saved = ctx->get_saved_variables();
        auto opt = [](const at::Tensor& t) { return t.defined() ? c10::optional<at::Tensor>(t) : c10::nullopt; };
        GradTuple g = hstu_dense_backward(grad_outputs[0], saved[0], saved[1], saved[2], opt(saved[3]), opt(saved[4]),
                                          ctx->saved_data["mask_type"].toInt(), ctx->saved_data["max_seq_len"].toInt(),
                                          ctx->saved_data["silu_scale"].toDouble());
        torch::autograd::tensor_list out(8);
        out[0] = std::get<0>(g);
        out[1] = std::get<1>(g);
        out[2] = std::get<2>(g);
        if (saved[4].defined()) out[4] = std::get<3>(g);
        return out;
    }
};

at::Tensor hstu_dense_autograd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const c10::optional<at::Tensor>& mask,
                               const c10::optional<at::Tensor>& attn_bias, int64_t mask_type, int64_t max_seq_len, double silu_scale) {
    return HstuDenseFunction::apply(q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale);
}

// ---------------------------------------------------------------------------------------------
// standalone bias producers (cust_op/framework/torch_plugin/torch_library/relative_attn_bias/)
// ---------------------------------------------------------------------------------------------
static void check_tensor_non_empty(const at::Tensor& t, const char* name) {   // common_utils.h:30-35
    TORCH_CHECK(t.defined(), name, " tensor must be defined");
    TORCH_CHECK(t.numel() > 0, name, " tensor must be non-empty");
    TORCH_CHECK(t.dim() > 0, name, " tensor must have non-zero dimensions");
}

static int32_t index_dtype(const at::Tensor& t, const char* name) {
    TORCH_CHECK(t.scalar_type() == at::kInt || t.scalar_type() == at::kLong, name, " dtype expect int32 or int64, but get ", t.scalar_type());
    return t.scalar_type() == at::kLong ? HSTU_I64 : HSTU_I32;
}

// relative_attn_bias_time_impl (relative_attn_bias_time.cpp:29-62); the repeat of the reference's wrapper is part of the kernel
static std::tuple<at::Tensor, at::Tensor> rab_time_impl(const at::Tensor& timestamps, const at::Tensor& weights, double bucket_divisor,
                                                        const char* op) {
    check_tensor_non_empty(timestamps, "timestampsConti");
    check_tensor_non_empty(weights, "timestampsWeightsConti");
    TORCH_CHECK(weights.dim() == 2, "timestampsWeightsConti must be 2D");
    TORCH_CHECK(timestamps.dim() == 2, "timestampsConti must be 2D");
    TORCH_CHECK(timestamps.device() == weights.device(), "timestamps and timestampsWeights must be on the same device");
    TORCH_CHECK(bucket_divisor > 0, "bucket_divisor must be positive");
    Holder h;
    auto ts = h.same(timestamps), w = h.same(weights);
    const int64_t n = w.size(0), cols = w.size(1), bs = ts.size(0), s = ts.size(1);
    TORCH_CHECK(s > 0 && s <= HSTU_RAB_MAX_SEQ_LEN, "timestamps size must be between 1 and ", HSTU_RAB_MAX_SEQ_LEN);
    hstu_rab_time_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(w, "timestamps_weights");
    p.index_type = index_dtype(ts, "timestamps");
    p.num_layers = (int32_t)n;
    p.batch = (int32_t)bs;
    p.seq_len = (int32_t)s;
    p.weight_cols = (int32_t)cols;
    p.bucket_divisor = (float)bucket_divisor;
    require_gpu(w, op);
    at::Tensor bounds = cols > 1 ? cached_bounds(cols - 1, bucket_divisor, w.device())
                                 : at::tensor({0.0f, std::numeric_limits<float>::infinity()}).to(w.device());
    auto out = at::empty({n, bs, 2 * s, 2 * s}, w.options());
    auto ids = at::empty({bs, s, s}, ts.options());
    p.timestamps = ts.const_data_ptr();
    p.weights = w.const_data_ptr();
    p.bucket_bounds = bounds.const_data_ptr<float>();
    p.rab_time_out = out.data_ptr();
    p.bucket_ts_out = ids.data_ptr();
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(w.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    const int rc = hstu_hip_rab_time(&p, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::", op, ": ", hstu_hip_last_error());
    return {out, ids};
}

// relative_attn_bias_time_backward_impl (relative_attn_bias_time.cpp:64-85)
at::Tensor relative_attn_bias_time_backward(const at::Tensor& rab_time_grad, const at::Tensor& bucket_timestamps, int64_t num_buckets) {
    check_tensor_non_empty(rab_time_grad, "rabTimeGrad");
    check_tensor_non_empty(bucket_timestamps, "bucketTimestamps");
    TORCH_CHECK(rab_time_grad.dim() == 4, "rabTimeGrad must be 4D");
    Holder h;
    auto g = h.same(rab_time_grad), ids = h.same(bucket_timestamps);
    const int64_t n = g.size(0), bs = g.size(1), sx2 = g.size(2), s = sx2 / 2;
    TORCH_CHECK(g.size(3) == sx2 && sx2 % 2 == 0 && ids.numel() == bs * s * s,
                "Sequence len mismatch between grad(_, _, ", sx2, ", ", g.size(3), ") and bucket_timestamps of ", ids.numel(), " elements");
    hstu_rab_time_bwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(g, "rab_time_grad");
    p.index_type = index_dtype(ids, "bucket_timestamps");
    p.num_layers = (int32_t)n;
    p.batch = (int32_t)bs;
    p.seq_len = (int32_t)s;
    p.num_buckets = (int32_t)num_buckets;
    require_gpu(g, "relative_attn_bias_time_backward");
    auto out = at::empty({n, num_buckets > 0 ? num_buckets : 0}, g.options().dtype(at::kFloat));
    p.grad = g.const_data_ptr();
    p.bucket_ts = ids.const_data_ptr();
    p.grad_weights = out.data_ptr<float>();
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(g.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    const int rc = hstu_hip_rab_time_backward(&p, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::relative_attn_bias_time_backward: ", hstu_hip_last_error());
    return g.scalar_type() == at::kFloat ? out : out.to(g.scalar_type());
}

at::Tensor relative_attn_bias_time(const at::Tensor& timestamps, const at::Tensor& weights, double bucket_divisor) {
    return std::get<0>(rab_time_impl(timestamps, weights, bucket_divisor, "relative_attn_bias_time"));
}

std::vector<at::Tensor> relative_attn_bias_time_with_index(const at::Tensor& timestamps, const at::Tensor& weights, double bucket_divisor) {
    auto r = rab_time_impl(timestamps, weights, bucket_divisor, "relative_attn_bias_time_with_index");
    return {std::get<0>(r), std::get<1>(r)};
}

// autograd of relative_attn_bias_time, as the reference's RelativeAttnBiasTime (relative_attn_bias_time.cpp:101-131)
class RabTimeFunction : public torch::autograd::Function<RabTimeFunction> {
public:
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, const at::Tensor& timestamps, const at::Tensor& weights, double bucket_divisor) {
        at::AutoDispatchBelowADInplaceOrView guard;
        auto r = rab_time_impl(timestamps, weights, bucket_divisor, "relative_attn_bias_time");
        ctx->save_for_backward({std::get<1>(r)});
        ctx->saved_data["num_buckets"] = weights.size(1);
        return std::get<0>(r);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list grad_outputs) {
        auto ids = ctx->get_saved_variables()[0];
        auto gw = relative_attn_bias_time_backward(grad_outputs[0], ids, ctx->saved_data["num_buckets"].toInt());
        return {at::Tensor(), gw, at::Tensor()};
    }
};

at::Tensor relative_attn_bias_time_autograd(const at::Tensor& timestamps, const at::Tensor& weights, double bucket_divisor) {
    return RabTimeFunction::apply(timestamps, weights, bucket_divisor);
}

// relative_attn_bias_pos_forward (relative_attn_bias_pos.cpp:22-43)
at::Tensor relative_attn_bias_pos(const at::Tensor& rel_pos_bias, const at::Tensor& identity, at::IntArrayRef past_valid_lens) {
    check_tensor_non_empty(rel_pos_bias, "relPosBias");
    check_tensor_non_empty(identity, "identity");
    TORCH_CHECK(rel_pos_bias.dim() == 2, "Invalid rel_pos_bias shape.");
    TORCH_CHECK(identity.dim() == 2, "Invalid identity shape.");
    TORCH_CHECK(rel_pos_bias.device() == identity.device(), "relPosBias and identity must be on the same device");
    TORCH_CHECK(identity.scalar_type() == rel_pos_bias.scalar_type(), "Mismatch data type of identity and rel_pos_bias.");
    Holder h;
    auto rel = h.same(rel_pos_bias), ident = h.same(identity);
    const int64_t sx2 = rel.size(0), bs = (int64_t)past_valid_lens.size();
    TORCH_CHECK(rel.size(1) == sx2 && ident.size(0) == sx2 && ident.size(1) == sx2, "Mismatch sequence len of rel_pos_bias and identity.");
    const int32_t dt = io_dtype(rel, "rel_pos_bias");
    require_gpu(rel, "relative_attn_bias_pos");
    auto out = at::empty({bs, sx2, sx2}, rel.options());
    std::vector<int64_t> lens(past_valid_lens.begin(), past_valid_lens.end());
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(rel.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    const int rc = hstu_hip_rab_pos(dt, (int32_t)sx2, rel.const_data_ptr(), ident.const_data_ptr(), lens.data(), (int32_t)bs, out.data_ptr(),
                                    (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::relative_attn_bias_pos: ", hstu_hip_last_error());
    return out;
}

// ---------------------------------------------------------------------------------------------
// norm_multiply_dropout (cust_op/framework/torch_plugin/torch_library/norm_multiply_dropout/norm_multiply_dropout.cpp)
// ---------------------------------------------------------------------------------------------
static void nmd_check_params(const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight, const at::Tensor& bias, double eps,
                             double dropout_ratio) {   // check_params, norm_multiply_dropout.cpp:150-171
    TORCH_CHECK(x.dim() == 2, "norm_multiply_dropout input x must be 2D");
    TORCH_CHECK(u.dim() == 2, "norm_multiply_dropout input u must be 2D");
    TORCH_CHECK(weight.dim() == 1, "norm_multiply_dropout input weight must be 1D");
    TORCH_CHECK(bias.dim() == 1, "norm_multiply_dropout input bias must be 1D");
    const auto d0 = x.size(0), d1 = x.size(1);
    TORCH_CHECK(d0 == u.size(0), "param input x dim0: ", d0, " is not equal to u dim0: ", u.size(0));
    TORCH_CHECK(d1 == u.size(1), "param input x dim1: ", d1, " is not equal to u dim1: ", u.size(1));
    TORCH_CHECK(d1 == weight.size(0) && weight.size(0) == bias.size(0), "param input x dim1: ", d1, ", weight dim0: ", weight.size(0),
                ", bias dim0:", bias.size(0), " must be same but not equal.");
    TORCH_CHECK(d0 >= 1 && d0 <= HSTU_NMD_MAX_ROWS, "x dim0 must in range:[1,", HSTU_NMD_MAX_ROWS, "].");
    TORCH_CHECK(d1 == 512 || d1 == 1024, "x dim1 must equal with ", 512, " or ", 1024);
    TORCH_CHECK(eps >= 1e-10 && eps <= 1e-4, "eps must in range:[", 1e-10, ",", 1e-4, "].");
    TORCH_CHECK(dropout_ratio >= 0.0 && dropout_ratio <= 1.0, "dropout_ratio must in range:[", 0.0, ",", 1.0, "].");
    TORCH_CHECK(u.scalar_type() == x.scalar_type() && weight.scalar_type() == x.scalar_type() && bias.scalar_type() == x.scalar_type(),
                "u, weight and bias must have the dtype of x");
}

// norm_multiply_dropout_impl_npu (norm_multiply_dropout.cpp:69-94): {result, mean, var, drop_mask}
static std::vector<at::Tensor> nmd_forward_impl(const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight, const at::Tensor& bias,
                                                double eps, double dropout_ratio) {
    Holder h;
    auto dx = h.same(x), du = h.same(u), dw = h.same(weight), db = h.same(bias);
    hstu_nmd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(dx, "x");
    p.rows = dx.size(0);
    p.cols = (int32_t)dx.size(1);
    p.eps = (float)eps;
    p.dropout_ratio = (float)dropout_ratio;
    require_gpu(dx, "norm_multiply_dropout");
    const bool drop = std::fabs(dropout_ratio) > 1e-10;
    auto out = at::empty_like(dx);
    auto mean = at::empty({dx.size(0)}, dx.options().dtype(at::kFloat));
    auto var = at::empty({dx.size(0)}, dx.options().dtype(at::kFloat));
    at::Tensor mask;
    if (drop) {
        mask = at::empty({(dx.numel() + 127) / 128 * 16}, dx.options().dtype(at::kByte));
        auto gen = at::detail::getDefaultCPUGenerator();
        std::lock_guard<std::mutex> lock(gen.mutex());
        p.seed = at::check_generator<at::CPUGeneratorImpl>(gen)->random64();
    } else {
        mask = at::empty({1}, dx.options().dtype(at::kByte));
    }
    p.x = dx.const_data_ptr();
    p.u = du.const_data_ptr();
    p.weight = dw.const_data_ptr();
    p.bias = db.const_data_ptr();
    p.out = out.data_ptr();
    p.mean = mean.data_ptr<float>();
    p.var = var.data_ptr<float>();
    p.drop_mask = mask.data_ptr<uint8_t>();
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dx.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    const int rc = hstu_hip_norm_multiply_dropout(&p, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::norm_multiply_dropout: ", hstu_hip_last_error());
    return {out, mean, var, mask};
}

// norm_multiply_dropout_backward_impl_npu (norm_multiply_dropout.cpp:97-111): {d_x, d_u, d_weight, d_bias}
static std::vector<at::Tensor> nmd_backward_impl(const at::Tensor& d_out, const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight,
                                                 const at::Tensor& bias, const at::Tensor& mean, const at::Tensor& var, const at::Tensor& mask,
                                                 double eps, double dropout_ratio) {
    Holder h;
    auto dy = h.same(d_out), dx = h.same(x), du = h.same(u), dw = h.same(weight), db = h.same(bias), dm = h.same(mean), dv = h.same(var), dk = h.same(mask);
    TORCH_CHECK(dy.sizes() == dx.sizes() && dy.scalar_type() == dx.scalar_type(), "d_out must have the shape and dtype of x");
    hstu_nmd_bwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(dx, "x");
    p.rows = dx.size(0);
    p.cols = (int32_t)dx.size(1);
    p.eps = (float)eps;
    p.dropout_ratio = (float)dropout_ratio;
    require_gpu(dx, "norm_multiply_dropout");
    auto gx = at::empty_like(dx), gu = at::empty_like(dx);
    auto gw = at::empty({dx.size(1)}, dx.options().dtype(at::kFloat)), gb = at::empty({dx.size(1)}, dx.options().dtype(at::kFloat));
    p.d_out = dy.const_data_ptr();
    p.x = dx.const_data_ptr();
    p.u = du.const_data_ptr();
    p.weight = dw.const_data_ptr();
    p.bias = db.const_data_ptr();
    p.mean = dm.const_data_ptr<float>();
    p.var = dv.const_data_ptr<float>();
    p.drop_mask = dk.const_data_ptr<uint8_t>();
    p.d_x = gx.data_ptr();
    p.d_u = gu.data_ptr();
    p.d_weight = gw.data_ptr<float>();
    p.d_bias = gb.data_ptr<float>();
    uint64_t ws_bytes = 0;
    int rc = hstu_hip_norm_multiply_dropout_backward_get_workspace_size(&p, &ws_bytes);
    TORCH_CHECK(rc == HSTU_OK, "mxrec::norm_multiply_dropout: ", hstu_hip_last_error());
    auto ws = at::empty({(int64_t)ws_bytes}, dx.options().dtype(at::kByte));
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dx.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    rc = hstu_hip_norm_multiply_dropout_backward(&p, ws.data_ptr(), ws_bytes, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::norm_multiply_dropout: ", hstu_hip_last_error());
    return {gx, gu, gw, gb};
}

// NormMultiplyDropout (norm_multiply_dropout.cpp:114-148)
class NmdFunction : public torch::autograd::Function<NmdFunction> {
public:
    static torch::autograd::tensor_list forward(torch::autograd::AutogradContext* ctx, const at::Tensor& x, const at::Tensor& u,
                                                const at::Tensor& weight, const at::Tensor& bias, double eps, double dropout_ratio) {
        at::AutoDispatchBelowADInplaceOrView guard;
        auto outs = nmd_forward_impl(x, u, weight, bias, eps, dropout_ratio);
        ctx->save_for_backward({x, u, weight, bias, outs[1], outs[2], outs[3]});
        ctx->saved_data["eps"] = eps;
        ctx->saved_data["dropout_ratio"] = dropout_ratio;
        return {outs[0]};
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list grad_outputs) {
        auto s = ctx->get_saved_variables();
        auto g = nmd_backward_impl(grad_outputs[0], s[0], s[1], s[2], s[3], s[4], s[5], s[6], ctx->saved_data["eps"].toDouble(),
                                   ctx->saved_data["dropout_ratio"].toDouble());
        // the parameter gradients are accumulated in fp32 and handed over in the parameters' dtype
        return {g[0], g[1], g[2].to(s[2].scalar_type()), g[3].to(s[3].scalar_type()), at::Tensor(), at::Tensor()};
    }
};

std::vector<at::Tensor> norm_multiply_dropout(const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight, const at::Tensor& bias, double eps,
                                              double dropout_ratio) {
    nmd_check_params(x, u, weight, bias, eps, dropout_ratio);
    return NmdFunction::apply(x, u, weight, bias, eps, dropout_ratio);
}

// the two halves as plain ops (no counterpart in the reference's registrations, which expose the pair only through autograd)
std::vector<at::Tensor> norm_multiply_dropout_forward(const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight, const at::Tensor& bias,
                                                      double eps, double dropout_ratio) {
    nmd_check_params(x, u, weight, bias, eps, dropout_ratio);
    return nmd_forward_impl(x, u, weight, bias, eps, dropout_ratio);
}
std::vector<at::Tensor> norm_multiply_dropout_backward(const at::Tensor& d_out, const at::Tensor& x, const at::Tensor& u, const at::Tensor& weight,
                                                       const at::Tensor& bias, const at::Tensor& mean, const at::Tensor& var, const at::Tensor& mask,
                                                       double eps, double dropout_ratio) {
    nmd_check_params(x, u, weight, bias, eps, dropout_ratio);
    return nmd_backward_impl(d_out, x, u, weight, bias, mean, var, mask, eps, dropout_ratio);
}

// ---------------------------------------------------------------------------------------------
// in_linear_silu, forward (cust_op/framework/torch_plugin/torch_library/in_linear_silu/in_linear_silu.cpp:34-117)
// ---------------------------------------------------------------------------------------------
std::vector<at::Tensor> distance_in_linear_silu(const at::Tensor& x, const at::Tensor& weight, const at::Tensor& bias, at::IntArrayRef split_list) {
    // IsValidShape, in_linear_silu.cpp:34-66
    check_tensor_non_empty(x, "x");
    check_tensor_non_empty(weight, "weight");
    TORCH_CHECK(x.dim() == 2, "x must be 2D");
    TORCH_CHECK(weight.dim() == 2, "weight must be 2D");
    TORCH_CHECK(split_list.size() == 4, "splitList must have 4 elements.");
    int64_t total = 0;
    for (int i = 0; i < 4; i++) {
        TORCH_CHECK(split_list[i] >= 16 && split_list[i] <= 8192 && split_list[i] % 16 == 0, "uvqk dim must in range[16, 8192] and multiples of 16.");
        total += split_list[i];
    }
    const auto k = x.size(1), n = weight.size(0), m = x.size(0);
    TORCH_CHECK(k >= 16 && k <= 8192 && k % 16 == 0, "x dim[1] must in range[16, 8192] and multiples of 16.");
    TORCH_CHECK(n >= 64 && n <= 32768 && n % 16 == 0, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    TORCH_CHECK(total == n, "weight_dim[0] must equal to sum(splitList).");
    TORCH_CHECK(weight.size(1) == k, "weight dim[1] must equal to x dim[1].");
    TORCH_CHECK(n % (4 * k) == 0, "weight dim[0] must be a multiple of 4 x dim[1]");
    if (bias.defined()) {
        check_tensor_non_empty(bias, "bias");
        TORCH_CHECK(bias.dim() == 1, "bias must be 1D");
        TORCH_CHECK(bias.size(0) == n, "bias dim[0] must equal to weight dim[0].");
    }
    TORCH_CHECK(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16, "x dtype expect float16 or bfloat16, but get ", x.scalar_type());
    TORCH_CHECK(weight.scalar_type() == x.scalar_type(), "weight must have the dtype of x");
    Holder h;
    auto dx = h.same(x), dw = h.same(weight);
    at::Tensor db;
    if (bias.defined()) db = h.same(bias.to(at::kFloat));
    hstu_in_linear_silu_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(dx, "x");
    p.m = m;
    p.k = (int32_t)k;
    p.n = (int32_t)n;
    require_gpu(dx, "distance_in_linear_silu");
    std::vector<at::Tensor> outs;
    for (int i = 0; i < 4; i++) {
        p.split[i] = (int32_t)split_list[i];
        outs.push_back(at::empty({m, split_list[i]}, dx.options()));
        p.out[i] = outs.back().data_ptr();
    }
    outs.push_back(at::empty({m, n}, dx.options()));
    p.linear_output = outs.back().data_ptr();
    p.x = dx.const_data_ptr();
    p.weight = dw.const_data_ptr();
    p.bias = db.defined() ? db.const_data_ptr<float>() : nullptr;
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dx.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    const int rc = hstu_hip_in_linear_silu(&p, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::distance_in_linear_silu: ", hstu_hip_last_error());
    return outs;
}

// in_linear_silu_backward (in_linear_silu.cpp:68-95 IsValidShapeBackward, :121-163 RunInLinearSiluBackward)
static void in_linear_silu_check(const at::Tensor& x, const at::Tensor& weight, const at::Tensor& bias, at::IntArrayRef split_list) {
    // IsValidShape, in_linear_silu.cpp:34-66
    check_tensor_non_empty(x, "x");
    check_tensor_non_empty(weight, "weight");
    TORCH_CHECK(x.dim() == 2, "x must be 2D");
    TORCH_CHECK(weight.dim() == 2, "weight must be 2D");
    TORCH_CHECK(split_list.size() == 4, "splitList must have 4 elements.");
    int64_t total = 0;
    for (int i = 0; i < 4; i++) {
        TORCH_CHECK(split_list[i] >= 16 && split_list[i] <= 8192 && split_list[i] % 16 == 0, "uvqk dim must in range[16, 8192] and multiples of 16.");
        total += split_list[i];
    }
    const auto k = x.size(1), n = weight.size(0);
    TORCH_CHECK(k >= 16 && k <= 8192 && k % 16 == 0, "x dim[1] must in range[16, 8192] and multiples of 16.");
    TORCH_CHECK(n >= 64 && n <= 32768 && n % 16 == 0, "weight dim[0] must in range[64, 32768] and multiples of 16.");
    TORCH_CHECK(total == n, "weight_dim[0] must equal to sum(splitList).");
    TORCH_CHECK(weight.size(1) == k, "weight dim[1] must equal to x dim[1].");
    TORCH_CHECK(n % (4 * k) == 0, "weight dim[0] must be a multiple of 4 x dim[1]");
    if (bias.defined()) {
        check_tensor_non_empty(bias, "bias");
        TORCH_CHECK(bias.dim() == 1, "bias must be 1D");
        TORCH_CHECK(bias.size(0) == n, "bias dim[0] must equal to weight dim[0].");
    }
    TORCH_CHECK(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16, "x dtype expect float16 or bfloat16, but get ", x.scalar_type());
    TORCH_CHECK(weight.scalar_type() == x.scalar_type(), "weight must have the dtype of x");
}

std::vector<at::Tensor> in_linear_silu_backward(const at::Tensor& x, const at::Tensor& weight, const c10::optional<at::Tensor>& bias,
                                                const at::Tensor& user_grad, const at::Tensor& value_grad, const at::Tensor& query_grad,
                                                const at::Tensor& key_grad, const at::Tensor& linear_output, at::IntArrayRef split_list) {
    const at::Tensor b = bias.has_value() ? bias.value() : at::Tensor();
    in_linear_silu_check(x, weight, b, split_list);
    const at::Tensor* grads[4] = {&user_grad, &value_grad, &query_grad, &key_grad};
    const char* names[4] = {"user_grad", "value_grad", "query_grad", "key_grad"};
    const auto m = x.size(0), k = x.size(1), n = weight.size(0);
    for (int i = 0; i < 4; i++) {
        check_tensor_non_empty(*grads[i], names[i]);
        TORCH_CHECK(grads[i]->dim() == 2, names[i], " must be 2D");
        TORCH_CHECK(grads[i]->size(1) == split_list[i], "user_grad, value_grad, query_grad, key_grad dim[1] must be equal to splitList.");
        TORCH_CHECK(grads[i]->size(0) == m, "user_grad, value_grad, query_grad, key_grad linear_output dim[0] must equal to x dim[0].");
        TORCH_CHECK(grads[i]->scalar_type() == x.scalar_type(), names[i], " must have the dtype of x");
    }
    check_tensor_non_empty(linear_output, "linear_output");
    TORCH_CHECK(linear_output.dim() == 2, "linear_output must be 2D");
    TORCH_CHECK(linear_output.size(0) == m, "user_grad, value_grad, query_grad, key_grad linear_output dim[0] must equal to x dim[0].");
    TORCH_CHECK(linear_output.size(1) == n, "linear_output dim[1] must equal to weight dim[0].");
    TORCH_CHECK(linear_output.scalar_type() == x.scalar_type(), "linear_output must have the dtype of x");
    Holder h;
    auto dx = h.same(x), dw = h.same(weight), dl = h.same(linear_output);
    require_gpu(dx, "in_linear_silu_backward");
    hstu_in_linear_silu_bwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.dtype = io_dtype(dx, "x");
    p.grad_dtype = p.dtype;   // the reference's wrapper hands x_grad and weight_grad back in the dtype of x and weight (:158)
    p.m = m;
    p.k = (int32_t)k;
    p.n = (int32_t)n;
    for (int i = 0; i < 4; i++) {
        p.split[i] = (int32_t)split_list[i];
        p.grad[i] = h.same(*grads[i]).const_data_ptr();
    }
    p.x = dx.const_data_ptr();
    p.weight = dw.const_data_ptr();
    p.linear_output = dl.const_data_ptr();
    auto x_grad = at::empty_like(dx), weight_grad = at::empty_like(dw);
    at::Tensor bias_grad32;
    if (b.defined()) bias_grad32 = at::empty({n}, dx.options().dtype(at::kFloat));
    p.x_grad = x_grad.data_ptr();
    p.weight_grad = weight_grad.data_ptr();
    p.bias_grad = bias_grad32.defined() ? bias_grad32.data_ptr<float>() : nullptr;
    uint64_t ws_bytes = 0;
    int rc = hstu_hip_in_linear_silu_backward_get_workspace_size(&p, &ws_bytes);
    TORCH_CHECK(rc == HSTU_OK, "mxrec::in_linear_silu_backward: ", hstu_hip_last_error());
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dx.device());
    auto ws = at::empty({(int64_t)ws_bytes}, dx.options().dtype(at::kByte));
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    rc = hstu_hip_in_linear_silu_backward(&p, ws.data_ptr(), ws_bytes, (void*)stream.stream());
    TORCH_CHECK(rc == HSTU_OK, "mxrec::in_linear_silu_backward: ", hstu_hip_last_error());
    at::Tensor bias_grad;
    if (b.defined()) bias_grad = bias_grad32.to(b.scalar_type());
    return {x_grad, weight_grad, bias_grad, at::Tensor()};
}

// in_linear_silu: the forward with the backward attached (RunInLinearSiluFunction, in_linear_silu.cpp:165-197)
class InLinearSiluFunction : public torch::autograd::Function<InLinearSiluFunction> {
public:
    static torch::autograd::tensor_list forward(torch::autograd::AutogradContext* ctx, const at::Tensor& x, const at::Tensor& weight,
                                                const at::Tensor& bias, at::IntArrayRef split_list) {
        at::AutoDispatchBelowADInplaceOrView guard;
        auto outs = distance_in_linear_silu(x, weight, bias, split_list);
        ctx->save_for_backward({x, weight, bias, outs[4]});
        ctx->saved_data["splitList"] = c10::List<int64_t>(split_list);
        return outs;
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list grad_outputs) {
        auto s = ctx->get_saved_variables();
        auto split = ctx->saved_data["splitList"].toIntVector();
        // an output that took no part in the loss arrives undefined: its gradient is zero
        for (int i = 0; i < 4; i++)
            if (!grad_outputs[i].defined()) grad_outputs[i] = at::zeros({s[0].size(0), split[i]}, s[0].options());
        return in_linear_silu_backward(s[0], s[1], s[2].defined() ? c10::optional<at::Tensor>(s[2]) : c10::nullopt, grad_outputs[0],
                                       grad_outputs[1], grad_outputs[2], grad_outputs[3], s[3], split);
    }
};

std::vector<at::Tensor> in_linear_silu(const at::Tensor& x, const at::Tensor& weight, const at::Tensor& bias, at::IntArrayRef split_list) {
    return InLinearSiluFunction::apply(x, weight, bias, split_list);
}

TORCH_LIBRARY_FRAGMENT(mxrec, m) {
    m.def("hstu_jagged.equal(Tensor q, "
          "                  Tensor k, "
          "                  Tensor v, "
          "                  Tensor? mask=None, "
          "                  Tensor? attn_bias=None, "
          "                  int mask_type=0, "
          "                  int max_seq_len=0, "
          "                  float silu_scale=0.0, "
          "                  Tensor seq_offset=None, "
          "                  Tensor? num_context=None, "
          "                  Tensor? num_target=None, "
          "                  int? target_group_size=0, "
          "                  float? alpha=1.0, "
          "                  bool deterministic=False) -> Tensor");
    m.def("hstu_jagged.delta(Tensor q, "
          "                  Tensor k, "
          "                  Tensor v, "
          "                  Tensor? mask=None, "
          "                  Tensor? attn_bias=None, "
          "                  int mask_type=0, "
          "                  int max_seq_len=0, "
          "                  int max_seq_len_k=0, "
          "                  float silu_scale=0.0, "
          "                  Tensor seq_offset=None, "
          "                  Tensor seq_offset_k=None, "
          "                  Tensor? num_context=None, "
          "                  Tensor? num_target=None, "
          "                  int? target_group_size=0, "
          "                  float? alpha=1.0, "
          "                  bool deterministic=False) -> Tensor");
    // schemas of hstu_jagged.cpp:202-215,232-247
    m.def("hstu_jagged_backward.equal(Tensor grad, "
          "                           Tensor q, "
          "                           Tensor k, "
          "                           Tensor v, "
          "                           Tensor? mask=None, "
          "                           Tensor? attn_bias=None, "
          "                           int mask_type=0, "
          "                           int max_seq_len=0, "
          "                           float silu_scale=0.0, "
          "                           Tensor seq_offset=None, "
          "                           Tensor? num_context=None, "
          "                           Tensor? num_target=None, "
          "                           int? target_group_size=0,"
          "                           float? alpha=1.0) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("hstu_jagged_backward.delta(Tensor grad, "
          "                           Tensor q, "
          "                           Tensor k, "
          "                           Tensor v, "
          "                           Tensor? mask=None, "
          "                           Tensor? attn_bias=None, "
          "                           int mask_type=0, "
          "                           int max_seq_len=0, "
          "                           int max_seq_len_k=0, "
          "                           float silu_scale=0.0, "
          "                           Tensor seq_offset=None, "
          "                           Tensor seq_offset_k=None, "
          "                           Tensor? num_context=None, "
          "                           Tensor? num_target=None, "
          "                           int? target_group_size=0,"
          "                           float? alpha=1.0) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("hstu_paged(Tensor q, "
          "           Tensor k, "
          "           Tensor v, "
          "           Tensor kv_cache=None, "
          "           Tensor? mask=None, "
          "           Tensor? attn_bias=None,"
          "           int mask_type=0, "
          "           int max_seq_len=0, "
          "           int max_seq_len_k=0, "
          "           float silu_scale=0.0, "
          "           Tensor seq_offset=None, "
          "           Tensor seq_offset_k=None, "
          "           Tensor seq_offset_t=None, "
          "           Tensor page_offsets=None, "
          "           Tensor page_ids=None, "
          "           Tensor last_page_len=None, "
          "           Tensor num_target=None, "
          "           int target_group_size=0, "
          "           float? alpha=1.0, "
          "           bool deterministic=False) -> Tensor");
    m.def("hstu_dense(Tensor q, "
          "           Tensor k, "
          "           Tensor v, "
          "           Tensor? mask=None, "
          "           Tensor? attn_bias=None, "
          "           int mask_type=0, "
          "           int max_seq_len=0, "
          "           float silu_scale=0.0) -> Tensor");
    m.def("hstu_dense_backward(Tensor grad, "
          "                    Tensor q, "
          "                    Tensor k, "
          "                    Tensor v, "
          "                    Tensor? mask, "
          "                    Tensor? attn_bias, "
          "                    int mask_type=0, "
          "                    int max_seq_len=0, "
          "                    float silu_scale=0.0) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("relative_attn_bias_pos(Tensor rel_pos_bias, "
          "                       Tensor identity, "
          "                       int[] past_valid_lens"
          "                       ) -> Tensor");
    m.def("relative_attn_bias_time(Tensor timestamps, "
          "                        Tensor timestamps_weights, "
          "                        float bucket_divisor"
          "                        ) -> Tensor");
    m.def("relative_attn_bias_time_backward(Tensor rab_time_grad, "
          "                                 Tensor bucket_timestamps, "
          "                                 int num_buckets"
          "                                 ) -> Tensor");
    m.def("relative_attn_bias_time_with_index(Tensor timestamps, "
          "                                   Tensor timestamps_weights, "
          "                                   float bucket_divisor"
          "                                   ) -> Tensor[]");
    // schemas of in_linear_silu.cpp:202-210
    m.def("distance_in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> Tensor[]");
    m.def("in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> Tensor[]");
    m.def("in_linear_silu_backward("
          "Tensor x, Tensor weight, Tensor ? bias,"
          "Tensor user_grad, Tensor value_grad, Tensor query_grad, Tensor key_grad,"
          "Tensor linear_output,"
          "int[] attr_dict) -> Tensor[]");
    m.def("norm_multiply_dropout(Tensor x, Tensor u, Tensor weight, Tensor bias, float eps, float dropout_ratio) -> "
          "Tensor[]");
    // no counterpart in the reference:
    m.def("norm_multiply_dropout_forward(Tensor x, Tensor u, Tensor weight, Tensor bias, float eps, float dropout_ratio) -> Tensor[]");
    m.def("norm_multiply_dropout_backward(Tensor d_out, Tensor x, Tensor u, Tensor weight, Tensor bias, Tensor mean, Tensor var, Tensor mask, "
          "float eps, float dropout_ratio) -> Tensor[]");
    m.def("hstu_jagged_table_bias(Tensor q, Tensor k, Tensor v, Tensor? pos_table=None, Tensor? ts_table=None, "
          "Tensor? timestamps=None, Tensor? attn_bias=None, int mask_type=0, int max_seq_len=0, int max_seq_len_k=0, "
          "float silu_scale=0.0, Tensor seq_offset=None, Tensor seq_offset_k=None, Tensor? num_context=None, "
          "Tensor? num_target=None, int? target_group_size=0, float? alpha=1.0, float bucket_divisor=0.301) -> Tensor");
    m.def("hstu_paged_fp8(Tensor q, Tensor k, Tensor v, Tensor kv_cache=None, Tensor kv_scales=None, Tensor? mask=None, "
          "Tensor? attn_bias=None, int mask_type=0, int max_seq_len=0, int max_seq_len_k=0, float silu_scale=0.0, "
          "Tensor seq_offset=None, Tensor seq_offset_k=None, Tensor seq_offset_t=None, Tensor page_offsets=None, "
          "Tensor page_ids=None, Tensor last_page_len=None, Tensor num_target=None, int target_group_size=0, "
          "float? alpha=1.0, bool deterministic=False) -> Tensor");
    m.def("hstu_time_bucket_bounds(int num_buckets=128, float bucket_divisor=0.301) -> Tensor", &hstu_time_bucket_bounds);
}

#define HSTU_IMPLS(m)                                                         \
    m.impl("hstu_jagged.equal", TORCH_FN(hstu_jagged_equal));                 \
    m.impl("hstu_jagged.delta", TORCH_FN(hstu_jagged_delta));                 \
    m.impl("hstu_jagged_backward.equal", TORCH_FN(hstu_jagged_backward_equal)); \
    m.impl("hstu_jagged_backward.delta", TORCH_FN(hstu_jagged_backward_delta)); \
    m.impl("hstu_paged", TORCH_FN(hstu_paged));                               \
    m.impl("hstu_dense", TORCH_FN(hstu_dense));                               \
    m.impl("hstu_dense_backward", TORCH_FN(hstu_dense_backward));             \
    m.impl("hstu_jagged_table_bias", TORCH_FN(hstu_jagged_table_bias));       \
    m.impl("hstu_paged_fp8", TORCH_FN(hstu_paged_fp8));                       \
    m.impl("relative_attn_bias_pos", TORCH_FN(relative_attn_bias_pos));       \
    m.impl("relative_attn_bias_time", TORCH_FN(relative_attn_bias_time));     \
    m.impl("relative_attn_bias_time_backward", TORCH_FN(relative_attn_bias_time_backward)); \
    m.impl("relative_attn_bias_time_with_index", TORCH_FN(relative_attn_bias_time_with_index)); \
    m.impl("norm_multiply_dropout_forward", TORCH_FN(norm_multiply_dropout_forward));           \
    m.impl("distance_in_linear_silu", TORCH_FN(distance_in_linear_silu));                       \
    m.impl("in_linear_silu_backward", TORCH_FN(in_linear_silu_backward));                       \
    m.impl("norm_multiply_dropout_backward", TORCH_FN(norm_multiply_dropout_backward));

// ROCm tensors dispatch on the CUDA key.  The CPU key runs the same host checks and then
// reports that there is no CPU implementation.
TORCH_LIBRARY_IMPL(mxrec, CUDA, m) { HSTU_IMPLS(m) }
TORCH_LIBRARY_IMPL(mxrec, CPU, m) { HSTU_IMPLS(m) }
// differentiable entry of the jagged op (reference: TORCH_LIBRARY_IMPL(mxrec, AutogradPrivateUse1, ...), hstu_jagged.cpp:352-356)
TORCH_LIBRARY_IMPL(mxrec, AutogradCUDA, m) {
    m.impl("hstu_jagged.equal", TORCH_FN(hstu_jagged_equal_autograd));
    m.impl("hstu_jagged.delta", TORCH_FN(hstu_jagged_delta_autograd));
    m.impl("hstu_dense", TORCH_FN(hstu_dense_autograd));
    m.impl("relative_attn_bias_time", TORCH_FN(relative_attn_bias_time_autograd));   // relative_attn_bias_time.cpp:143-146
}
// norm_multiply_dropout is registered under the device key and the Autograd key with one function, like the reference
// (norm_multiply_dropout.cpp:185-192): the checks, then the autograd Function
TORCH_LIBRARY_IMPL(mxrec, CUDA, m) { m.impl("norm_multiply_dropout", TORCH_FN(norm_multiply_dropout)); }
TORCH_LIBRARY_IMPL(mxrec, CPU, m) { m.impl("norm_multiply_dropout", TORCH_FN(norm_multiply_dropout)); }
TORCH_LIBRARY_IMPL(mxrec, Autograd, m) { m.impl("norm_multiply_dropout", TORCH_FN(norm_multiply_dropout)); }
// in_linear_silu exists only as the differentiable entry (in_linear_silu.cpp:218-227); without autograd it is the forward
TORCH_LIBRARY_IMPL(mxrec, CUDA, m) { m.impl("in_linear_silu", TORCH_FN(distance_in_linear_silu)); }
TORCH_LIBRARY_IMPL(mxrec, CPU, m) { m.impl("in_linear_silu", TORCH_FN(distance_in_linear_silu)); }
TORCH_LIBRARY_IMPL(mxrec, AutogradCUDA, m) { m.impl("in_linear_silu", TORCH_FN(in_linear_silu)); }

}  // namespace mxrec_hstu
