#include "linear.h"

#include <hip/hip_runtime_api.h>
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <algorithm>
#include <mutex>

#include "kernels.h"

namespace tq {

Policy& policy() {
    static Policy p;
    return p;
}

int* policy_field(const std::string& name) {
    Policy& p = policy();
    if (name == "skinny") return &p.skinny;
    if (name == "library") return &p.library;
    if (name == "fused") return &p.fused;
    if (name == "prune_last") return &p.prune_last;
    if (name == "packed") return &p.packed;
    if (name == "mid") return &p.mid;
    if (name == "keep_rows") return &p.keep_rows;
    if (name == "decode_mfma") return &p.decode_mfma;
    if (name == "prefill_mfma") return &p.prefill_mfma;
    return nullptr;
}

int skinny_max_rows() {
    static int n = K::skinny_max_rows.raw();
    return n;
}

int mid_max_rows() {
    static int n = K::mid_max_rows.raw();
    return n;
}

OwnedPtr make_owned(int dtype, const std::vector<int64_t>& dims) {
    OwnedPtr o = std::make_shared<Owned>();
    o->t.dtype = dtype;
    o->t.ndim = (int)dims.size();
    if (dims.size() > 6) raise(TQE_ERR_ARGUMENT, "tensors of %zu dimensions are not supported (6 at most)", dims.size());
    for (size_t i = 0; i < dims.size(); ++i) o->t.shape[i] = dims[i];
    o->mem.allocate(o->t.bytes());
    o->t.data = o->mem.data();
    return o;
}

OwnedPtr make_owned(int dtype, std::initializer_list<int64_t> dims) { return make_owned(dtype, std::vector<int64_t>(dims)); }

Weight make_weight(OwnedPtr rows, int parts, bool rows_needed, hipStream_t stream) {
    Weight w;
    const Tensor& t = rows->t;
    if (t.ndim != 2) raise(TQE_ERR_WEIGHTS, "a product's weight must have two dimensions, got %s", t.describe().c_str());
    w.n = t.shape[0];
    w.k = t.shape[1];
    w.parts = parts;
    w.dtype = t.dtype;
    w.rows = rows;
    const Policy& p = policy();
    if (p.packed && p.skinny && t.dtype == BF16 && !null_device() && w.k % 32 == 0 && w.n % parts == 0) {
        const int64_t per = w.n / parts, tiles = (per + 15) / 16;
        w.packed = make_owned(BF16, {parts * tiles, w.k / 32, 64, 8});
        K::pack_weight(t.data, w.packed->t.data, (int)w.n, (int)w.k, parts, stream);
        if (!p.keep_rows && !rows_needed && p.mid && p.skinny) {
            stream_synchronize(stream);         // the packing kernel has read the rows
            w.rows = nullptr;
        }
    }
    return w;
}

bool fusable(int64_t x_rows, const Weight& w, bool adds) {
    const Policy& p = policy();
    return p.fused && p.skinny && x_rows <= skinny_max_rows() && w.dtype == BF16 && w.k % 32 == 0 && (!adds || w.n % 4 == 0);
}

bool leaves_sums(int64_t x_rows, const Weight& w) {
    const Policy& p = policy();
    return p.mid && w.packed && w.dtype == BF16 && x_rows > skinny_max_rows() && x_rows <= mid_max_rows();
}

void classify_step(StepContext& c, int64_t hidden) {
    const Policy& p = policy();
    c.fuse_small = p.fused && c.act_dtype == BF16 && c.all_decode && c.n_tokens <= skinny_max_rows() && hidden % 32 == 0;
    c.fuse_mid = p.mid && c.act_dtype == BF16 && c.n_tokens > skinny_max_rows() && c.n_tokens <= mid_max_rows();
}

static bool skinny_ok(const Tensor& x, const Weight& w) {
    return policy().skinny && x.dtype == BF16 && w.dtype == BF16 && x.shape[1] % 32 == 0 && x.shape[0] <= skinny_max_rows();
}

static bool mid_ok(const Tensor& x, const Weight& w) { return x.dtype == BF16 && leaves_sums(x.shape[0], w); }

// pointer and packed flag of a product's weight for the few-row kernels
static const void* few_ptr(const Weight& w, int* packed) {
    if (w.packed) { *packed = 1; return w.packed->t.data; }
    if (!w.rows) raise(TQE_ERR_STATE, "a weight has neither rows nor a packed copy");
    *packed = 0;
    return w.rows->t.data;
}

static void k_fused_store(StepContext& c, const Tensor& x, const int32_t* rows, const LazyNorm* norm, const Weight& w, Tensor& out) {
    int packed = 0;
    const void* wp = few_ptr(w, &packed);
    K::fused_store(x.data, rows, norm ? (const float*)norm->ss.data : nullptr, norm ? norm->n_ss : 0, norm ? norm->eps : 0.f, wp, packed,
                   out.data, out.dtype, (int)out.shape[0], (int)w.n, (int)w.k, c.stream);
}

static void k_fused_gated(StepContext& c, const Tensor& x, const LazyNorm* norm, const Weight& w, Tensor& out) {
    int packed = 0;
    const void* wp = few_ptr(w, &packed);
    K::fused_gated(x.data, norm ? (const float*)norm->ss.data : nullptr, norm ? norm->n_ss : 0, norm ? norm->eps : 0.f, wp, packed, out.data,
                   (int)out.shape[0], (int)w.n, (int)w.k, c.stream);
}

// the product through the kernel for mid-sized steps; leave: its sums where it cuts K into pieces
static Product k_mid_store(StepContext& c, const Tensor& x, const Weight& w, int out_dtype, bool leave, Tensor* out) {
    const int64_t m = x.shape[0];
    const int splits = K::mid_splits.raw((int)w.n, (int)w.k, 0);
    Product p;
    Tensor scratch;
    if (splits > 1) scratch = c.alloc(F32, {splits, m, w.n});
    if (leave && splits > 1) {
        K::mid_store(x.data, w.packed->t.data, nullptr, out_dtype, (int)m, (int)w.n, (int)w.k, scratch.data, 0, c.stream);
        p.is_sums = true;
        p.sums.sums = scratch;
        p.sums.dtype = out_dtype;
        return p;
    }
    p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
    K::mid_store(x.data, w.packed->t.data, p.t.data, out_dtype, (int)m, (int)w.n, (int)w.k, scratch.data, 1, c.stream);
    return p;
}

static void k_mid_gated(StepContext& c, const Tensor& x, const Weight& w, Tensor& out) {
    const int64_t m = x.shape[0];
    const int splits = K::mid_splits.raw((int)w.n, (int)w.k, 1);
    Tensor scratch;
    if (splits > 1) scratch = c.alloc(F32, {splits, m, w.n});
    K::mid_gated(x.data, w.packed->t.data, out.data, (int)m, (int)w.n, (int)w.k, scratch.data, c.stream);
}

static void k_gemm(StepContext& c, const Tensor& x, const Tensor& w, const Tensor* bias, Tensor& out) {
    const int m = (int)x.shape[0], k = (int)x.shape[1], n = (int)w.shape[0];
    const int bias_dt = bias ? bias->dtype : 0;
    const size_t need = K::gemm_scratch_bytes.raw(x.dtype, w.dtype, bias_dt, out.dtype, m, n, k);
    void* scratch = need ? c.ws->alloc(need) : nullptr;
    K::gemm(x.data, x.dtype, w.data, w.dtype, bias ? bias->data : nullptr, bias_dt, out.data, out.dtype, m, n, k, scratch, c.stream);
}

Product linear(StepContext& c, const Tensor& x, const Weight& w, const Tensor* bias, int out_dtype, bool leave_sums, Tensor* out) {
    if (x.ndim != 2 || x.shape[1] != w.k)
        raise(TQE_ERR_ARGUMENT, "linear: x has %lld columns but the weight has %lld", (long long)(x.ndim == 2 ? x.shape[1] : -1), (long long)w.k);
    const int64_t m = x.shape[0];
    const bool both_bf16 = x.dtype == BF16 && w.dtype == BF16;
    Product p;
    if (both_bf16 && !bias) {
        if (skinny_ok(x, w)) {
            p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
            k_fused_store(c, x, nullptr, nullptr, w, p.t);
            return p;
        }
        if (mid_ok(x, w)) return k_mid_store(c, x, w, out_dtype, leave_sums, out);
        if (!w.rows && m > mid_max_rows() && policy().library && !null_device()) {
            // the rows were given up and this is a prompt: the rows come back for the length of this product (the weight
            // read and written once more, against reading it once per 128 rows of x)
            Tensor rows = c.alloc(BF16, {w.n, w.k});
            K::unpack_weight(w.packed->t.data, rows.data, (int)w.n, (int)w.k, w.parts, c.stream);
            p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
            library_gemm(x, rows, p.t, c.stream);
            return p;
        }
        if (!w.rows) {
            // every number of rows through the own kernels, in pieces that each stream the weight once
            p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
            const int64_t step = mid_max_rows();
            for (int64_t r = 0; r < m; r += step) {
                Tensor xs = x.slice(r, std::min(m, r + step)), os = p.t.slice(r, std::min(m, r + step));
                if (xs.shape[0] <= skinny_max_rows()) k_fused_store(c, xs, nullptr, nullptr, w, os);
                else k_mid_store(c, xs, w, out_dtype, false, &os);
            }
            return p;
        }
        if (policy().library && m > skinny_max_rows() && !null_device()) {
            p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
            library_gemm(x, w.rows->t, p.t, c.stream);
            return p;
        }
    }
    if (!w.rows)
        raise(TQE_ERR_STATE, "linear: this weight's rows were given up (policy keep_rows); only bfloat16 products without a bias take its packed copy");
    p.t = out ? *out : c.alloc(out_dtype, {m, w.n});
    k_gemm(c, x, w.rows->t, bias, p.t);
    return p;
}

Tensor gated_silu_linear(StepContext& c, const Tensor& x, const Weight& w) {
    const int64_t m = x.shape[0], inter = w.n / 2;
    Tensor act = c.alloc(x.dtype, {m, inter});
    if (skinny_ok(x, w)) { k_fused_gated(c, x, nullptr, w, act); return act; }
    if (mid_ok(x, w)) { k_mid_gated(c, x, w, act); return act; }
    if (!w.rows && !(m > mid_max_rows() && policy().library && !null_device())) {
        const int64_t step = mid_max_rows();
        for (int64_t r = 0; r < m; r += step) {
            Tensor xs = x.slice(r, std::min(m, r + step)), os = act.slice(r, std::min(m, r + step));
            if (xs.shape[0] <= skinny_max_rows()) k_fused_gated(c, xs, nullptr, w, os);
            else k_mid_gated(c, xs, w, os);
        }
        return act;
    }
    Product both = linear(c, x, w, nullptr, x.dtype);
    K::swiglu(both.t.data, act.data, act.dtype, (int)m, (int)inter, c.stream);
    return act;
}

// The few-row kernel that adds to the stream keeps one block per tile of 16 features, a block stays on one compute
// unit, and a compute unit alone pulls about a 256th of what the memory gives when all of them pull.  Where the tiles
// fall badly on the units (the 320 tiles of a 5120-wide product on 256 units: a quarter of the units work twice as long
// as the others) the kernel that cuts K into pieces over all units is faster, in spite of the norm kernel that then
// has to add the pieces up.  Estimated from the shape alone, so a product takes one way whatever the batch.
static bool pieces_pay(const Weight& w) {
    if (!policy().mid || !w.packed || w.dtype != BF16 || w.k % 32 != 0) return false;
    const int units = compute_units();
    if (units <= 0 || K::mid_splits.raw((int)w.n, (int)w.k, 0) <= 1) return false;
    const int blocks = K::fused_residual_parts.raw((int)w.n, (int)w.k);
    const double rounds = (double)((blocks + units - 1) / units);
    const double covered = (double)blocks / (rounds * units);
    const double bytes = 2.0 * (double)w.n * (double)w.k, rate = 6.5e6;          // bytes a microsecond with every unit pulling
    const double fused_us = bytes / (covered * rate), pieces_us = bytes / (0.85 * rate) + 6.0;
    return pieces_us + 2.0 < fused_us;
}

void add_product(StepContext& c, Stream& stream, const Tensor& x, const Weight& w) {
    if (x.shape[0] > skinny_max_rows() || pieces_pay(w)) {
        const bool leave = stream.next_norm && stream.next_norm->takes_partial_sums();
        Product p = k_mid_store(c, x, w, BF16, leave, nullptr);
        stream.pending = p.is_sums ? Pending::of(p.sums) : Pending::of(p.t);
        stream.invalidate();
        return;
    }
    const Norm* norm = stream.next_norm && stream.next_norm->foldable() ? stream.next_norm : nullptr;
    int packed = 0;
    const void* wp = few_ptr(w, &packed);
    const int parts = K::fused_residual_parts.raw((int)w.n, (int)w.k);
    if (stream.ss_buffer.defined() && stream.ss_buffer.numel() < (int64_t)parts * 16)
        raise(TQE_ERR_STATE, "the stream's buffer for sums of squares holds %lld values, %d pieces of 16 are written",
              (long long)stream.ss_buffer.numel(), parts);
    K::fused_residual(x.data, wp, packed, (float*)stream.h.data, norm ? norm->fold_weight()->data : nullptr, stream.xw_buffer.data,
                      (float*)stream.ss_buffer.data, (int)x.shape[0], (int)w.n, (int)w.k, c.stream);
    stream.n_ss = parts;
    stream.xw_for = norm;
    stream.pending = Pending();
}

void k_add_rmsnorm(StepContext& c, float* h, const Pending& delta, const Tensor& weight, float eps, const int32_t* rows, int64_t n_rows,
                   int64_t src_rows, Tensor& out, bool write_back) {
    const int hidden = (int)weight.shape[0];
    if (!rows && src_rows != n_rows) raise(TQE_ERR_ARGUMENT, "add_rmsnorm: %lld input rows but %lld output rows", (long long)src_rows, (long long)n_rows);
    if (delta.kind == Pending::Sums) {
        const PartialSums& s = delta.s;
        if (s.dtype != out.dtype || s.rows() != src_rows || s.cols() != hidden)
            raise(TQE_ERR_ARGUMENT, "add_rmsnorm: the update's sums are [%lld, %lld] of %s, wanted [%lld, %d] of %s", (long long)s.rows(),
                  (long long)s.cols(), dtype_name(s.dtype), (long long)src_rows, hidden, dtype_name(out.dtype));
        K::add_rmsnorm_sums(h, (const float*)s.sums.data, (int)s.sums.shape[0], (int)src_rows, out.dtype, weight.data, weight.dtype, eps, rows,
                            (int)n_rows, hidden, out.data, write_back ? 1 : 0, c.stream);
        return;
    }
    const void* d = delta.kind == Pending::Plain ? delta.t.data : nullptr;
    if (d && (delta.t.dtype != out.dtype || delta.t.shape[0] != src_rows || delta.t.cols() != hidden))
        raise(TQE_ERR_ARGUMENT, "add_rmsnorm: the update is %s, wanted [%lld, %d] of %s", delta.t.describe().c_str(), (long long)src_rows, hidden,
              dtype_name(out.dtype));
    K::add_rmsnorm(h, d, out.dtype, weight.data, weight.dtype, eps, rows, (int)n_rows, hidden, out.data, write_back ? 1 : 0, c.stream);
}

void k_gather_rows(StepContext& c, const Tensor& src, const int32_t* rows, int64_t n_rows, Tensor& out) {
    if (out.shape[0] != n_rows || out.row_bytes() != src.row_bytes())
        raise(TQE_ERR_ARGUMENT, "gather_rows: %s from %s", out.describe().c_str(), src.describe().c_str());
    K::gather_rows(src.data, rows, (int)n_rows, (long long)src.row_bytes(), out.data, c.stream);
}

// ---- the library's product ---------------------------------------------------------------------
namespace {

struct Library {
    std::mutex mutex;
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    size_t workspace_bytes = (size_t)128 << 20;
    struct Plan {
        hipblasLtMatmulDesc_t desc = nullptr;
        hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
        hipblasLtMatmulAlgo_t algo;
    };
    std::map<std::tuple<int64_t, int64_t, int64_t, int>, Plan> plans;
};

Library& library() {
    static Library lib;
    return lib;
}

void lt_check(hipblasStatus_t s, const char* what) {
    if (s != HIPBLAS_STATUS_SUCCESS) raise(TQE_ERR_DEVICE, "hipBLASLt: %s failed with status %d", what, (int)s);
}

}  // namespace

namespace {

// the plan of a shape, with the library's proposals for it (the first that fits is the plan's kernel until tuning says otherwise)
Library::Plan& plan_for(Library& lib, int64_t m, int64_t n, int64_t k, int out_dtype, std::vector<hipblasLtMatmulHeuristicResult_t>* proposals, int want) {
    if (!lib.handle) {
        lt_check(hipblasLtCreate(&lib.handle), "creating the handle");
        lib.workspace = device_malloc(lib.workspace_bytes);
    }
    const auto key = std::make_tuple(m, n, k, out_dtype);
    auto it = lib.plans.find(key);
    if (it != lib.plans.end() && !proposals) return it->second;
    // in the library's column-major terms: out^T [n, m] = w [n, k] (the k x n matrix, transposed) * x^T [k, m]
    Library::Plan fresh;
    Library::Plan& plan = it != lib.plans.end() ? it->second : fresh;
    if (it == lib.plans.end()) {
        lt_check(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "creating a product");
        const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
        lt_check(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)), "setting a product");
        lt_check(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)), "setting a product");
        lt_check(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, (uint64_t)k, (uint64_t)n, k), "describing the weight");
        lt_check(hipblasLtMatrixLayoutCreate(&plan.b, HIP_R_16BF, (uint64_t)k, (uint64_t)m, k), "describing x");
        lt_check(hipblasLtMatrixLayoutCreate(&plan.c, out_dtype == F32 ? HIP_R_32F : HIP_R_16BF, (uint64_t)n, (uint64_t)m, n), "describing the output");
    }
    hipblasLtMatmulPreference_t pref;
    lt_check(hipblasLtMatmulPreferenceCreate(&pref), "creating a preference");
    lt_check(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &lib.workspace_bytes, sizeof(lib.workspace_bytes)),
             "setting the workspace");
    std::vector<hipblasLtMatmulHeuristicResult_t> found((size_t)want);
    int n_found = 0;
    const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(lib.handle, plan.desc, plan.a, plan.b, plan.c, plan.c, pref, want, found.data(), &n_found);
    hipblasLtMatmulPreferenceDestroy(pref);
    lt_check(st, "choosing a kernel");
    found.resize((size_t)std::max(n_found, 0));
    found.erase(std::remove_if(found.begin(), found.end(), [&](const hipblasLtMatmulHeuristicResult_t& r) { return r.workspaceSize > lib.workspace_bytes; }),
                found.end());
    if (found.empty()) raise(TQE_ERR_DEVICE, "hipBLASLt has no kernel for a product of %lld x %lld x %lld", (long long)m, (long long)n, (long long)k);
    if (it == lib.plans.end()) {
        plan.algo = found[0].algo;
        it = lib.plans.emplace(key, plan).first;
    }
    if (proposals) *proposals = found;
    return it->second;
}

void run_plan(Library& lib, const Library::Plan& plan, const hipblasLtMatmulAlgo_t& algo, const void* w, const void* x, void* out, hipStream_t stream) {
    const float alpha = 1.f, beta = 0.f;
    lt_check(hipblasLtMatmul(lib.handle, plan.desc, &alpha, w, plan.a, x, plan.b, &beta, out, plan.c, out, plan.c, &algo, lib.workspace,
                             lib.workspace_bytes, stream),
             "the product");
}

}  // namespace

void library_gemm(const Tensor& x, const Tensor& w, Tensor& out, hipStream_t stream) {
    const int64_t m = x.shape[0], k = x.shape[1], n = w.shape[0];
    if (x.dtype != BF16 || w.dtype != BF16 || w.shape[1] != k || out.shape[0] != m || out.cols() != n || (out.dtype != BF16 && out.dtype != F32))
        raise(TQE_ERR_ARGUMENT, "library product: %s times %s^T into %s", x.describe().c_str(), w.describe().c_str(), out.describe().c_str());
    if (m == 0) return;
    Library& lib = library();
    std::lock_guard<std::mutex> lock(lib.mutex);
    const Library::Plan& plan = plan_for(lib, m, n, k, out.dtype, nullptr, 4);
    run_plan(lib, plan, plan.algo, w.data, x.data, out.data, stream);
}

double library_tune(int64_t m, int64_t n, int64_t k, int out_dtype, hipStream_t stream) {
    if (m < 1 || n < 1 || k < 1 || null_device()) return 0.0;
    Library& lib = library();
    std::lock_guard<std::mutex> lock(lib.mutex);
    std::vector<hipblasLtMatmulHeuristicResult_t> proposals;
    Library::Plan& plan = plan_for(lib, m, n, k, out_dtype, &proposals, 8);
    {
        // beside what the library proposes for the shape, every kernel it has for these types that takes the shape
        std::vector<hipblasLtMatmulHeuristicResult_t> all;
        const hipDataType out_type = out_dtype == F32 ? HIP_R_32F : HIP_R_16BF;
        if (hipblaslt_ext::getAllAlgos(lib.handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, HIPBLAS_OP_T, HIPBLAS_OP_N, HIP_R_16BF, HIP_R_16BF, out_type,
                                       out_type, HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
            const float one = 1.f, zero = 0.f;
            for (hipblasLtMatmulHeuristicResult_t& r : all) {
                size_t ws = 0;
                if (hipblaslt_ext::matmulIsAlgoSupported(lib.handle, plan.desc, &one, plan.a, plan.b, &zero, plan.c, plan.c, r.algo, ws) ==
                        HIPBLAS_STATUS_SUCCESS && ws <= lib.workspace_bytes)
                    proposals.push_back(r);
            }
        }
    }
    // operands of the right sizes with values as the model's are (zeros would let the matrix cores run cooler and faster
    // than real data does): the weight's and x's memory is filled with the random-weights stream
    Buffer x((size_t)m * k * 2), w((size_t)n * k * 2), out((size_t)m * n * dtype_size(out_dtype));
    K::random_normal(x.data(), BF16, (long long)(m * k), 0x1234u, 1.0f, 0, stream);
    K::random_normal(w.data(), BF16, (long long)(n * k), 0x5678u, 0.02f, 0, stream);
    hipEvent_t a = nullptr, b = nullptr;
    hip_check(hipEventCreate(&a), "creating an event");
    hip_check(hipEventCreate(&b), "creating an event");
    // one run each (after one that does not count), then the eight fastest again, ten runs each: what is kept is the
    // fastest of those
    auto time_one = [&](size_t i, int warm, int reps) -> double {
        const float alpha = 1.f, beta = 0.f;
        for (int r = 0; r < warm; ++r)
            if (hipblasLtMatmul(lib.handle, plan.desc, &alpha, w.data(), plan.a, x.data(), plan.b, &beta, out.data(), plan.c, out.data(), plan.c,
                                &proposals[i].algo, lib.workspace, lib.workspace_bytes, stream) != HIPBLAS_STATUS_SUCCESS)
                return 1e30;
        hip_check(hipEventRecord(a, stream), "recording an event");
        for (int r = 0; r < reps; ++r)
            if (hipblasLtMatmul(lib.handle, plan.desc, &alpha, w.data(), plan.a, x.data(), plan.b, &beta, out.data(), plan.c, out.data(), plan.c,
                                &proposals[i].algo, lib.workspace, lib.workspace_bytes, stream) != HIPBLAS_STATUS_SUCCESS)
                return 1e30;
        hip_check(hipEventRecord(b, stream), "recording an event");
        hip_check(hipEventSynchronize(b), "waiting for the device");
        float ms = 0.f;
        hip_check(hipEventElapsedTime(&ms, a, b), "reading a time");
        return ms * 1000.0 / reps;
    };
    std::vector<std::pair<double, size_t>> first;
    for (size_t i = 0; i < proposals.size(); ++i) first.push_back({time_one(i, 1, 1), i});
    std::sort(first.begin(), first.end());
    double best = 1e30;
    size_t best_i = first.empty() ? 0 : first[0].second;
    for (size_t r = 0; r < first.size() && r < 8; ++r) {
        if (first[r].first >= 1e29) break;
        const double us = time_one(first[r].second, 1, 10);
        if (us < best) { best = us; best_i = first[r].second; }
    }
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    if (best < 1e29) plan.algo = proposals[best_i].algo;
    return best;
}

void library_release() {
    Library& lib = library();
    std::lock_guard<std::mutex> lock(lib.mutex);
    for (auto& e : lib.plans) {
        hipblasLtMatmulDescDestroy(e.second.desc);
        hipblasLtMatrixLayoutDestroy(e.second.a);
        hipblasLtMatrixLayoutDestroy(e.second.b);
        hipblasLtMatrixLayoutDestroy(e.second.c);
    }
    lib.plans.clear();
    if (lib.workspace) { device_free(lib.workspace, false); lib.workspace = nullptr; }
    if (lib.handle) { hipblasLtDestroy(lib.handle); lib.handle = nullptr; }
}

}  // namespace tq
