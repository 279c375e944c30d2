// torch extension `blockAttention`: the reference's operator surface
// (csrc/sparseBlockedAttention.cpp:118-136) on top of the C ABI in
// include/blocked_attention.h.  Host code only; compiled by the host compiler.
//
//   sparseBlockedGEMM(mat1, mat2, mat1Accum?, mat2Accum?, outAccum?, MList?, NList?, KList?,
//                     transpose1, transpose2) -> Tensor [H, Dout]
//   sparseBlockedSoftmax(src, rowList?, colList?, srcAccum?) -> Tensor [H, Dsrc]
//
// Additions that keep the reference behaviour when left at their defaults:
//   sparseBlockedSoftmaxScaled(src, rowList, colList, srcAccum?, scale)
//   sparseBlockedGEMMSoftmax(mat1, mat2, ..., scale, out_fp32)   fused pair, forward only
//
// Every precondition the reference leaves to assert() is a TORCH_CHECK here.
// The tensors are used as device memory only; all work happens in
// libblockedattn_hip.so on the current HIP stream.  Scheduling costs one host
// synchronisation: reading the plan summary, which carries Dout (needed to
// allocate the result) and the device-side metadata verdict.  The layers and
// heads of a model call these operators many times with the SAME metadata
// tensors, so the last few schedules are kept, keyed by the identity and the
// version counter of every metadata tensor: a repeated call launches its
// kernels at once.  set_schedule_cache(0) turns that off (needed only by a
// caller that rewrites metadata tensors behind PyTorch's back, through raw
// pointers, which the version counters cannot see).
#include <array>
#include <deque>
#include <memory>
#include <mutex>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include "blocked_attention.h"

namespace {

using torch::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;
using OptTensor = std::optional<Tensor>;

void *current_stream(const Tensor &t) { return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

void check_status(int st, const char *what) {
    TORCH_CHECK(st == BA_OK, what, ": ", ba_status_string(st), " (status ", st, ")");
}

int dtype_code(const Tensor &t, const char *name) {
    switch (t.scalar_type()) {
        case at::kHalf: return BA_F16;
        case at::kBFloat16: return BA_BF16;
        case at::kFloat: return BA_F32;
        case at::kDouble: return BA_F64;
        case at::kByte: return BA_U8;
        case at::kChar: return BA_I8;
        case at::kShort: return BA_I16;
        case at::kInt: return BA_I32;
        case at::kLong: return BA_I64;
        default: TORCH_CHECK(false, name, ": dtype ", t.scalar_type(), " is not supported");
    }
    return -1;
}

void check_data(const Tensor &t, const char *name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

void check_meta(const Tensor &t, const char *name, const Tensor &like, int64_t n) {
    check_data(t, name);
    TORCH_CHECK(t.scalar_type() == at::kLong, name, " must be int64");
    TORCH_CHECK(t.device() == like.device(), name, " must be on the same device as the data");
    TORCH_CHECK(t.dim() == 1 && t.numel() == n, name, " must be 1-D with ", n, " entries, got ", t.sizes());
}

int64_t leading(const Tensor &t) {
    int64_t h = 1;
    for (int64_t d = 0; d + 1 < t.dim(); ++d) h *= t.size(d);
    return h;
}

struct Schedule;
// Schedules derived from one schedule (permuted shapes for the two GEMMs of the backward pass), made on first
// use and shared by every copy of the schedule, so that they live and die with its cache entry.
struct Derived {
    std::mutex mu;
    std::shared_ptr<Schedule> grad1, grad2;
};

struct Schedule {
    Tensor accum1, accum2, accumOut, M, N, K;
    Tensor plan;
    ba_plan_info info;
    std::shared_ptr<Derived> derived;
};

// ---------------------------------------------------------------- schedule cache
struct ScheduleKey {
    int kind = 0;                                   // 0 GEMM, 1 softmax
    int device = -1;
    std::array<const void *, 6> impl{};             // TensorImpl of each metadata tensor (nullptr: not given)
    std::array<int64_t, 6> version{};
    bool cacheable = true;
    bool operator==(const ScheduleKey &o) const {
        return kind == o.kind && device == o.device && impl == o.impl && version == o.version;
    }
};

ScheduleKey make_key(int kind, const Tensor &like, std::initializer_list<const OptTensor *> metas) {
    ScheduleKey k;
    k.kind = kind;
    k.device = like.device().index();
    size_t i = 0;
    for (const OptTensor *m : metas) {
        if (m->has_value() && (*m)->defined()) {
            if ((*m)->is_inference()) k.cacheable = false;      // no version counter to watch
            else { k.impl[i] = (*m)->unsafeGetTensorImpl(); k.version[i] = (int64_t)(*m)->_version(); }
        }
        ++i;
    }
    return k;
}

struct ScheduleCache {
    std::mutex mu;
    std::deque<std::pair<ScheduleKey, Schedule>> entries;       // most recent first; entries keep their tensors alive
    size_t capacity = 8;
    int64_t hits = 0, misses = 0;
};
ScheduleCache &cache() {
    static ScheduleCache c;
    return c;
}

bool cache_lookup(const ScheduleKey &key, Schedule &out) {
    ScheduleCache &c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.capacity == 0 || !key.cacheable) return false;
    for (auto it = c.entries.begin(); it != c.entries.end(); ++it) {
        if (it->first == key) {
            out = it->second;
            if (it != c.entries.begin()) {
                auto e = *it;
                c.entries.erase(it);
                c.entries.push_front(std::move(e));
            }
            ++c.hits;
            return true;
        }
    }
    ++c.misses;
    return false;
}

void cache_store(const ScheduleKey &key, const Schedule &s) {
    ScheduleCache &c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.capacity == 0 || !key.cacheable) return;
    c.entries.emplace_front(key, s);
    while (c.entries.size() > c.capacity) c.entries.pop_back();
}

void set_schedule_cache(int64_t capacity) {
    TORCH_CHECK(capacity >= 0 && capacity <= 1024, "schedule cache capacity must be in [0, 1024]");
    ScheduleCache &c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    c.capacity = (size_t)capacity;
    while (c.entries.size() > c.capacity) c.entries.pop_back();
}

std::vector<int64_t> schedule_cache_stats() {
    ScheduleCache &c = cache();
    std::lock_guard<std::mutex> lock(c.mu);
    return {c.hits, c.misses, (int64_t)c.entries.size(), (int64_t)c.capacity};
}

// Where a scheduler launch hands its summary to the host: BA_MAILBOX_BYTES of pinned, GPU-writable memory per
// calling thread (allocated at the thread's first schedule, kept for the life of the process) and a ticket that
// changes with every use.  The host then spins on the ticket instead of copying and synchronising the stream.
struct Mailbox {
    void *mem = nullptr;
    uint32_t ticket = 0;
    Mailbox() {
        if (hipHostMalloc(&mem, BA_MAILBOX_BYTES, hipHostMallocCoherent | hipHostMallocMapped | hipHostMallocPortable) != hipSuccess) mem = nullptr;
        else memset(mem, 0, BA_MAILBOX_BYTES);
    }
};
Mailbox &mailbox() {
    static thread_local Mailbox m;
    return m;
}

// The three metadata cases of the reference (cpp:17-44), resolved on the device.
Schedule schedule_gemm(const Tensor &like, const OptTensor &a1, const OptTensor &a2, const OptTensor &aO,
                       const OptTensor &M, const OptTensor &N, const OptTensor &K, bool use_cache = true) {
    const bool have_accum = a1.has_value() && a2.has_value() && aO.has_value();
    const bool have_lists = M.has_value() && N.has_value() && K.has_value();
    TORCH_CHECK(have_accum || have_lists,
                "sparseBlockedGEMM needs either (mat1Accum, mat2Accum, outAccum) or (MList, NList, KList)");
    Schedule s;
    const ScheduleKey key = make_key(0, like, {&a1, &a2, &aO, &M, &N, &K});
    if (use_cache && cache_lookup(key, s)) return s;
    s.derived = std::make_shared<Derived>();
    int64_t nseg;
    int mode;
    const auto opts = at::TensorOptions().dtype(at::kLong).device(like.device());
    if (have_lists) {
        nseg = M->numel();
        check_meta(*M, "MList", like, nseg); check_meta(*N, "NList", like, nseg); check_meta(*K, "KList", like, nseg);
        s.M = *M; s.N = *N; s.K = *K;
    }
    if (have_accum) {
        nseg = a1->numel() - 1;
        TORCH_CHECK(nseg >= 0, "prefix sums need at least one entry");
        check_meta(*a1, "mat1Accum", like, nseg + 1); check_meta(*a2, "mat2Accum", like, nseg + 1);
        check_meta(*aO, "outAccum", like, nseg + 1);
        if (have_lists) TORCH_CHECK(s.M.numel() == nseg, "lists and prefix sums disagree on the segment count");
        s.accum1 = *a1; s.accum2 = *a2; s.accumOut = *aO;
    }
    if (have_lists && have_accum) {
        mode = BA_META_GIVEN;
    } else if (have_lists) {
        mode = BA_META_FROM_LISTS;
        s.accum1 = at::empty({nseg + 1}, opts); s.accum2 = at::empty({nseg + 1}, opts);
        s.accumOut = at::empty({nseg + 1}, opts);
    } else {
        mode = BA_META_FROM_ACCUM;
        s.M = at::empty({nseg}, opts); s.N = at::empty({nseg}, opts); s.K = at::empty({nseg}, opts);
    }
    const size_t bytes = ba_plan_bytes(nseg);
    s.plan = at::empty({(int64_t)bytes}, at::TensorOptions().dtype(at::kByte).device(like.device()));
    void *stream = current_stream(like);
    Mailbox &mb = mailbox();
    int st;
    if (mb.mem) {
        const uint32_t ticket = ++mb.ticket ? mb.ticket : ++mb.ticket;       // never 0, the mailbox's first content
        check_status(ba_plan_gemm_notify(s.plan.data_ptr(), bytes, nseg, mode, s.M.data_ptr<int64_t>(),
                                         s.N.data_ptr<int64_t>(), s.K.data_ptr<int64_t>(), s.accum1.data_ptr<int64_t>(),
                                         s.accum2.data_ptr<int64_t>(), s.accumOut.data_ptr<int64_t>(), mb.mem, ticket,
                                         stream),
                     "ba_plan_gemm_notify");
        st = ba_plan_wait(mb.mem, ticket, &s.info, 60 * 1000 * 1000);
    } else {
        check_status(ba_plan_gemm(s.plan.data_ptr(), bytes, nseg, mode, s.M.data_ptr<int64_t>(),
                                  s.N.data_ptr<int64_t>(), s.K.data_ptr<int64_t>(), s.accum1.data_ptr<int64_t>(),
                                  s.accum2.data_ptr<int64_t>(), s.accumOut.data_ptr<int64_t>(), stream),
                     "ba_plan_gemm");
        st = ba_plan_read(s.plan.data_ptr(), &s.info, stream);
    }
    TORCH_CHECK(st != BA_ERR_BAD_METADATA, "segment metadata rejected: ", s.info.bad_segments,
                " segment(s) have negative, oversized or inconsistent shapes / prefix sums");
    check_status(st, "ba_plan_read");
    if (use_cache) cache_store(key, s);
    return s;
}

Schedule schedule_softmax(const Tensor &like, const Tensor &rows, const Tensor &cols, const OptTensor &accum) {
    Schedule s;
    const OptTensor rows_o(rows), cols_o(cols), none;
    const ScheduleKey key = make_key(1, like, {&rows_o, &cols_o, &accum, &none, &none, &none});
    if (cache_lookup(key, s)) return s;
    const int64_t nseg = rows.numel();
    check_meta(rows, "rowList", like, nseg); check_meta(cols, "colList", like, nseg);
    s.M = rows; s.N = cols;
    if (accum.has_value()) {
        check_meta(*accum, "srcAccum", like, nseg + 1);
        s.accumOut = *accum;
    } else {
        s.accumOut = at::empty({nseg + 1}, at::TensorOptions().dtype(at::kLong).device(like.device()));
    }
    const size_t bytes = ba_plan_bytes(nseg);
    s.plan = at::empty({(int64_t)bytes}, at::TensorOptions().dtype(at::kByte).device(like.device()));
    void *stream = current_stream(like);
    Mailbox &mb = mailbox();
    int st;
    if (mb.mem) {
        const uint32_t ticket = ++mb.ticket ? mb.ticket : ++mb.ticket;
        check_status(ba_plan_softmax_notify(s.plan.data_ptr(), bytes, nseg, rows.data_ptr<int64_t>(), cols.data_ptr<int64_t>(),
                                            s.accumOut.data_ptr<int64_t>(), accum.has_value() ? 1 : 0, mb.mem, ticket, stream),
                     "ba_plan_softmax_notify");
        st = ba_plan_wait(mb.mem, ticket, &s.info, 60 * 1000 * 1000);
    } else {
        check_status(ba_plan_softmax(s.plan.data_ptr(), bytes, nseg, rows.data_ptr<int64_t>(), cols.data_ptr<int64_t>(),
                                     s.accumOut.data_ptr<int64_t>(), accum.has_value() ? 1 : 0, stream),
                     "ba_plan_softmax");
        st = ba_plan_read(s.plan.data_ptr(), &s.info, stream);
    }
    TORCH_CHECK(st != BA_ERR_BAD_METADATA, "segment metadata rejected: ", s.info.bad_segments,
                " segment(s) have negative or oversized shapes or a prefix sum too small for them");
    check_status(st, "ba_plan_read");
    cache_store(key, s);
    return s;
}

// sparseBlockedGEMMLaunch (h:18; GEMM.cu:985-1033): result is always [H, Dout] in mat1's dtype.
Tensor gemm_launch(const Tensor &mat1, const Tensor &mat2, Schedule &s, bool t1, bool t2) {
    check_data(mat1, "mat1"); check_data(mat2, "mat2");
    TORCH_CHECK(mat1.scalar_type() == mat2.scalar_type(), "mat1 and mat2 must have the same dtype, got ",
                mat1.scalar_type(), " and ", mat2.scalar_type());
    TORCH_CHECK(mat1.device() == mat2.device(), "mat1 and mat2 must be on the same device");
    TORCH_CHECK(mat1.dim() >= 1 && mat2.dim() >= 1, "mat1 and mat2 need a last dimension");
    TORCH_CHECK(mat1.size(-1) == s.info.Dm1, "mat1.size(-1) = ", mat1.size(-1), " but the segments need ", s.info.Dm1);
    TORCH_CHECK(mat2.size(-1) == s.info.Dm2, "mat2.size(-1) = ", mat2.size(-1), " but the segments need ", s.info.Dm2);
    const int64_t H = leading(mat1);
    TORCH_CHECK(leading(mat2) == H, "mat1 and mat2 disagree on the number of heads");
    const int dt = dtype_code(mat1, "sparseBlockedGEMM");
    Tensor out = at::empty({H, s.info.Dout}, mat1.options());
    check_status(ba_varlen_gemm(s.plan.data_ptr(), &s.info, s.info.nseg, dt, mat1.data_ptr(), mat2.data_ptr(), out.data_ptr(), H,
                                s.info.Dm1, s.info.Dm2, s.info.Dout, t1, t2, current_stream(mat1)),
                 "ba_varlen_gemm");
    return out;
}

// The schedule of one of the two backward products of s (permuted metadata, given in both forms), made once and
// kept with s: it lives and dies with the forward schedule and takes no slot of the cache.
Schedule &derived_schedule(const Schedule &s, std::shared_ptr<Schedule> Derived::*slot, const Tensor &like,
                           const Tensor &a1, const Tensor &a2, const Tensor &aO, const Tensor &rows, const Tensor &cols,
                           const Tensor &reduce) {
    TORCH_CHECK(s.derived, "internal: schedule without a holder for derived schedules");
    std::lock_guard<std::mutex> lock(s.derived->mu);
    std::shared_ptr<Schedule> &p = (*s.derived).*slot;
    if (!p)
        p = std::make_shared<Schedule>(schedule_gemm(like, OptTensor(a1), OptTensor(a2), OptTensor(aO), OptTensor(rows),
                                                     OptTensor(cols), OptTensor(reduce), /*use_cache=*/false));
    return *p;
}

class SparseBlockedGEMM : public torch::autograd::Function<SparseBlockedGEMM> {
public:
    static variable_list forward(AutogradContext *ctx, const Tensor &mat1, const Tensor &mat2, const OptTensor &a1,
                                 const OptTensor &a2, const OptTensor &aO, const OptTensor &M, const OptTensor &N,
                                 const OptTensor &K, bool t1, bool t2) {
        check_data(mat1, "mat1"); check_data(mat2, "mat2");
        c10::hip::HIPGuardMasqueradingAsCUDA guard(mat1.device());
        Schedule s = schedule_gemm(mat1, a1, a2, aO, M, N, K);
        ctx->save_for_backward({mat1, mat2, s.accum1, s.accum2, s.accumOut, s.M, s.N, s.K});
        ctx->saved_data["transpose1"] = t1;
        ctx->saved_data["transpose2"] = t2;
        return {gemm_launch(mat1, mat2, s, t1, t2)};
    }

    // dA = dS B and dB = dS^T A as two more varlen GEMMs with permuted metadata
    // (cpp:52-72); like the reference, the gradient layouts are those of the
    // untransposed forward.
    static variable_list backward(AutogradContext *ctx, const variable_list &grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor grad = grads[0].contiguous();
        c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
        const Tensor mat1 = saved[0].to(grad.scalar_type()), mat2 = saved[1].to(grad.scalar_type());
        const Tensor &a1 = saved[2], &a2 = saved[3], &aO = saved[4], &M = saved[5], &N = saved[6], &K = saved[7];
        const bool t1 = ctx->saved_data["transpose1"].toBool(), t2 = ctx->saved_data["transpose2"].toBool();
        Tensor g1, g2;
        // dS and the saved operands are read as they lie: the products whose reduction runs over N or M take the
        // kernels for any layout and reduction length (two launches, like the reference)
        Schedule fwd = schedule_gemm(grad, a1, a2, aO, M, N, K);          // the forward's, from the cache
        Schedule &s1 = derived_schedule(fwd, &Derived::grad1, grad, aO, a2, a1, M, K, N);
        Schedule &s2 = derived_schedule(fwd, &Derived::grad2, grad, aO, a1, a2, N, K, M);
        // batches of short segments: both products as ONE launch where the library offers it (layouts of the
        // untransposed forward), else one call each
        bool done = false;
        if (!t1 && !t2 && grad.dim() >= 1 && grad.size(-1) == s1.info.Dm1 && mat2.size(-1) == s1.info.Dm2 &&
            grad.size(-1) == s2.info.Dm1 && mat1.size(-1) == s2.info.Dm2 && leading(mat1) == leading(grad) &&
            leading(mat2) == leading(grad) && (grad.scalar_type() == at::kHalf || grad.scalar_type() == at::kBFloat16)) {
            const int64_t H = leading(grad);
            g1 = at::empty({H, s1.info.Dout}, grad.options());
            g2 = at::empty({H, s2.info.Dout}, grad.options());
            const int st = ba_varlen_gemm_two(dtype_code(grad, "sparseBlockedGEMM backward"), H, s1.plan.data_ptr(), &s1.info,
                                              grad.data_ptr(), mat2.data_ptr(), g1.data_ptr(), s1.info.Dm1, s1.info.Dm2,
                                              s1.info.Dout, s2.plan.data_ptr(), &s2.info, grad.data_ptr(), mat1.data_ptr(),
                                              g2.data_ptr(), s2.info.Dm1, s2.info.Dm2, s2.info.Dout, current_stream(grad));
            if (st == BA_OK) done = true;
            else if (st != BA_ERR_UNSUPPORTED) check_status(st, "ba_varlen_gemm_two");
        }
        if (!done) {
            g1 = gemm_launch(grad, mat2, s1, false, !t2);
            g2 = gemm_launch(grad, mat1, s2, true, !t1);
        }
        return {g1.view_as(saved[0]), g2.view_as(saved[1]), Tensor(), Tensor(), Tensor(), Tensor(), Tensor(),
                Tensor(), Tensor(), Tensor()};
    }
};

class SparseBlockedSoftmax : public torch::autograd::Function<SparseBlockedSoftmax> {
public:
    static variable_list forward(AutogradContext *ctx, const Tensor &src, const OptTensor &rows,
                                 const OptTensor &cols, const OptTensor &accum, double scale) {
        TORCH_CHECK(rows.has_value() && cols.has_value(), "sparseBlockedSoftmax needs rowList and colList");
        check_data(src, "src");
        c10::hip::HIPGuardMasqueradingAsCUDA guard(src.device());
        Schedule s = schedule_softmax(src, *rows, *cols, accum);
        TORCH_CHECK(src.dim() >= 1 && src.size(-1) == s.info.Dout, "src.size(-1) = ", src.size(-1),
                    " but the segments need ", s.info.Dout);
        const int64_t H = leading(src);
        const int dt = dtype_code(src, "sparseBlockedSoftmax");
        Tensor out = at::empty({H, s.info.Dout}, src.options());
        check_status(ba_blocked_softmax(s.plan.data_ptr(), &s.info, s.info.nseg, dt, src.data_ptr(), out.data_ptr(), H,
                                        s.info.Dout, (float)scale, current_stream(src)),
                     "ba_blocked_softmax");
        ctx->save_for_backward({out, s.accumOut, s.M, s.N});
        ctx->saved_data["scale"] = scale;
        return {out};
    }

    static variable_list backward(AutogradContext *ctx, const variable_list &grads) {
        const auto saved = ctx->get_saved_variables();
        const Tensor grad = grads[0].contiguous();
        c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
        const Tensor y = saved[0].to(grad.scalar_type());
        Schedule s = schedule_softmax(grad, saved[2], saved[3], saved[1]);
        const int64_t H = leading(y);
        Tensor dx = at::empty_like(y);
        check_status(ba_blocked_softmax_backward(s.plan.data_ptr(), &s.info, s.info.nseg,
                                                 dtype_code(y, "softmax backward"),
                                                 y.data_ptr(), grad.data_ptr(), dx.data_ptr(), H, s.info.Dout,
                                                 (float)ctx->saved_data["scale"].toDouble(), current_stream(y)),
                     "ba_blocked_softmax_backward");
        return {dx, Tensor(), Tensor(), Tensor(), Tensor()};
    }
};

// ------------------------------------------------------------------ the ops
Tensor sparseBlockedGEMM_op(const Tensor &mat1, const Tensor &mat2, const OptTensor &mat1Accum,
                            const OptTensor &mat2Accum, const OptTensor &outAccum, const OptTensor &MList,
                            const OptTensor &NList, const OptTensor &KList, bool transpose1, bool transpose2) {
    return SparseBlockedGEMM::apply(mat1, mat2, mat1Accum, mat2Accum, outAccum, MList, NList, KList, transpose1,
                                    transpose2)[0];
}

Tensor sparseBlockedSoftmax_op(const Tensor &src, const OptTensor &rowList, const OptTensor &colList,
                               const OptTensor &srcAccum) {
    return SparseBlockedSoftmax::apply(src, rowList, colList, srcAccum, 1.0)[0];
}

Tensor sparseBlockedSoftmaxScaled_op(const Tensor &src, const OptTensor &rowList, const OptTensor &colList,
                                     const OptTensor &srcAccum, double scale) {
    return SparseBlockedSoftmax::apply(src, rowList, colList, srcAccum, scale)[0];
}

// Fused softmax(scale * A_g B_g^T): forward only, scores never leave registers.
Tensor sparseBlockedGEMMSoftmax_op(const Tensor &mat1, const Tensor &mat2, const OptTensor &mat1Accum,
                                   const OptTensor &mat2Accum, const OptTensor &outAccum, const OptTensor &MList,
                                   const OptTensor &NList, const OptTensor &KList, double scale, bool out_fp32) {
    check_data(mat1, "mat1"); check_data(mat2, "mat2");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(mat1.device());
    TORCH_CHECK(mat1.scalar_type() == mat2.scalar_type(), "mat1 and mat2 must have the same dtype");
    TORCH_CHECK(mat1.scalar_type() == at::kHalf || mat1.scalar_type() == at::kBFloat16,
                "the fused GEMM + softmax takes fp16 or bf16 operands");
    TORCH_CHECK(mat1.device() == mat2.device(), "mat1 and mat2 must be on the same device");
    Schedule s = schedule_gemm(mat1, mat1Accum, mat2Accum, outAccum, MList, NList, KList);
    TORCH_CHECK(mat1.size(-1) == s.info.Dm1 && mat2.size(-1) == s.info.Dm2,
                "operand sizes do not match the segments: need ", s.info.Dm1, " and ", s.info.Dm2);
    const int64_t H = leading(mat1);
    TORCH_CHECK(leading(mat2) == H, "mat1 and mat2 disagree on the number of heads");
    Tensor out = at::empty({H, s.info.Dout}, out_fp32 ? mat1.options().dtype(at::kFloat) : mat1.options());
    check_status(ba_gemm_softmax(s.plan.data_ptr(), &s.info, s.info.nseg, dtype_code(mat1, "fused"), mat1.data_ptr(),
                                 mat2.data_ptr(), out.data_ptr(), out_fp32 ? BA_F32 : dtype_code(mat1, "fused"), H,
                                 s.info.Dm1, s.info.Dm2, s.info.Dout, (float)scale, current_stream(mat1)),
                 "ba_gemm_softmax");
    return out;
}

// softmax(scale * Q_g K_g^T) V_g in one pass: forward only, the probabilities are never written.
// Q is the M x K operand of the segments, K and V are both N x K; the result has Q's shape.
Tensor sparseBlockedAttention_op(const Tensor &q, const Tensor &k, const Tensor &v, const OptTensor &mat1Accum,
                                 const OptTensor &mat2Accum, const OptTensor &outAccum, const OptTensor &MList,
                                 const OptTensor &NList, const OptTensor &KList, double scale) {
    check_data(q, "q"); check_data(k, "k"); check_data(v, "v");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    TORCH_CHECK(q.scalar_type() == k.scalar_type() && q.scalar_type() == v.scalar_type(),
                "q, k and v must have the same dtype");
    TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16,
                "the one-pass attention takes fp16 or bf16 operands");
    TORCH_CHECK(q.device() == k.device() && q.device() == v.device(), "q, k and v must be on the same device");
    Schedule s = schedule_gemm(q, mat1Accum, mat2Accum, outAccum, MList, NList, KList);
    TORCH_CHECK(q.size(-1) == s.info.Dm1 && k.size(-1) == s.info.Dm2 && v.size(-1) == s.info.Dm2,
                "operand sizes do not match the segments: need ", s.info.Dm1, " (q) and ", s.info.Dm2, " (k, v)");
    TORCH_CHECK(s.info.max_K <= 128, "the one-pass attention takes head dimensions up to 128, got ", s.info.max_K);
    const int64_t H = leading(q);
    TORCH_CHECK(leading(k) == H && leading(v) == H, "q, k and v disagree on the number of heads");
    Tensor out = at::empty({H, s.info.Dm1}, q.options());
    check_status(ba_varlen_attention(s.plan.data_ptr(), &s.info, s.info.nseg, dtype_code(q, "attention"), q.data_ptr(),
                                     k.data_ptr(), v.data_ptr(), out.data_ptr(), H, s.info.Dm1, s.info.Dm2,
                                     s.info.Dout, (float)scale, current_stream(q)),
                 "ba_varlen_attention");
    return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("sparseBlockedGEMM", &sparseBlockedGEMM_op, "sparseBlockedGEMM forward");
    m.def("sparseBlockedSoftmax", &sparseBlockedSoftmax_op, "sparseBlockedSoftmax forward");
    m.def("sparseBlockedSoftmaxScaled", &sparseBlockedSoftmaxScaled_op, "sparseBlockedSoftmax with a fused scale");
    m.def("sparseBlockedGEMMSoftmax", &sparseBlockedGEMMSoftmax_op, "fused sparseBlockedGEMM + softmax forward");
    m.def("sparseBlockedAttention", &sparseBlockedAttention_op, "softmax(scale q k^T) v per segment, one pass");
    m.def("set_schedule_cache", &set_schedule_cache, "number of schedules kept for repeated metadata (0 = off)");
    m.def("schedule_cache_stats", &schedule_cache_stats, "[hits, misses, entries, capacity]");
}
