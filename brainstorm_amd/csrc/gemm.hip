// dot_mm / dot_add_mm through hipBLASLt. The handler's matrices are row-major;
// hipBLASLt is column-major, so C = op(A) op(B) is issued as
// C^T = op(B)^T op(A)^T by swapping the operands. Descriptors and the algorithm
// chosen by the heuristic are cached per problem shape, because recurrent
// networks issue the same small product thousands of times per step. The cache
// holds the kMaxPlans most recently used shapes (workloads with varying batch or
// sequence lengths would otherwise grow it without limit).
//
// Optional (BSHIP_GEMM_AUTOTUNE=1): thin products (one side of the result at most 128 long: a batch of 100
// rows against a weight matrix) are where the library's heuristic is furthest from its own best kernel
// (measured on MI355X for 100x4000 . 4000x1000, launches back to back: first choice 18.1 us, best of the
// offered 14.1 us). With the switch on, the candidates for such a shape are timed once, on the caller's
// operands and a scratch result, when the shape is first seen outside a recording, and a candidate more than
// 5 % faster than the first choice replaces it. Off by default: in the network workloads measured here the
// trial's ranking did not carry over to the layers reliably (see fastest_candidate), and without it a shape
// runs the same kernel in every process.
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"
#include "window.h"

namespace bship {

namespace {

struct GemmPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    uint64_t last_use = 0;
};

typedef std::tuple<int, int, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int> GemmKey;   // ..., with bias

std::mutex g_gemm_mutex;
hipblasLtHandle_t g_handle = nullptr;
std::map<GemmKey, GemmPlan> g_plans;
constexpr size_t kMaxPlans = 512;
uint64_t g_use_counter = 0;
// The products' workspace is not a pool block: the first product may arrive while a step is being
// recorded, and blocks handed out then belong to that recording.
void* g_workspace = nullptr;
constexpr size_t kWorkspaceBytes = 64u << 20;

int blas_error(hipblasStatus_t s, const char* what) {
    return set_error(BSHIP_ERR_BLAS, "%s failed with hipblasStatus %d", what, static_cast<int>(s));
}

#define BSHIP_BLAS(call)                                       \
    do {                                                       \
        hipblasStatus_t _s = (call);                           \
        if (_s != HIPBLAS_STATUS_SUCCESS) return blas_error(_s, #call); \
    } while (0)

void destroy_plan(GemmPlan& p) {
    if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
    if (p.lb) hipblasLtMatrixLayoutDestroy(p.lb);
    if (p.lc) hipblasLtMatrixLayoutDestroy(p.lc);
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    p = GemmPlan();
}

// The operands of the call that creates a plan, for timing the candidates on them.
struct TuneOperands { const float* a; const float* b; const float* bias; };

// BSHIP_GEMM_AUTOTUNE: 0 or unset = the heuristic's first choice, 1 = timed choice, 2 = timed choice and a
// line on stderr per shape.
int tune_mode() {
    static const int mode = [] { const char* e = getenv("BSHIP_GEMM_AUTOTUNE"); return e && e[0] ? atoi(e) : 0; }();
    return mode;
}
bool tune_verbose() { return tune_mode() >= 2; }

// Index of the candidate that runs fastest: each is launched four times untimed and 32 times between two
// events on the library's stream, into a scratch result (the caller's result may be an accumulator). The
// heuristic's first choice is kept unless another candidate is more than 5 % faster.
// Candidates that need more workspace than the library keeps are skipped; if the scratch block or an
// event cannot be had, or a candidate fails, the heuristic's first choice stands.
int fastest_candidate(const GemmPlan& p, const hipblasLtMatmulHeuristicResult_t* res, int found, const float* a,
                      const float* b, const float* bias, int64_t c_elements) {
    void* scratch = nullptr;
    if (pool_alloc_raw(static_cast<size_t>(c_elements) * sizeof(float), &scratch) != 0 || scratch == nullptr) return 0;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int best = 0, fastest = 0;
    if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
        if (bias) (void)hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
        const float alpha = 1.0f, beta = 0.0f;
        float* c = static_cast<float*>(scratch);
        float best_ms = 1e30f, first_ms = 1e30f;
        hipStream_t stream = ctx().stream;
        for (int i = 0; i < found; ++i) {
            if (res[i].workspaceSize > kWorkspaceBytes) continue;
            bool ok = true;
            for (int r = 0; r < 36 && ok; ++r) {
                if (r == 4) (void)hipEventRecord(e0, stream);
                ok = hipblasLtMatmul(g_handle, p.desc, &alpha, a, p.la, b, p.lb, &beta, c, p.lc, c, p.lc, &res[i].algo,
                                     g_workspace, kWorkspaceBytes, stream) == HIPBLAS_STATUS_SUCCESS;
            }
            float ms = 1e30f;
            if (hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
                hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
                ok = false;
            if (i == 0 && ok) first_ms = ms;
            if (ok && ms < best_ms) { best_ms = ms; best = i; fastest = i; }
        }
        // Only a clear win replaces the first choice: the trial runs one product back to back on warm operands,
        // a layer runs it between other kernels, and candidates within a few per cent of each other in the
        // trial came out in either order there (an LSTM step with one stacked product per time step: 5.46 ms
        // with the first choices, 5.51-5.74 ms from process to process with the trial's winners by 1-2 %; the
        // recorded LSTM step through single operations 19.3 -> 18.0 ms with a winner by 3 %, 19.4 without it).
        if (best_ms > 0.95f * first_ms) best = 0;
        if (tune_verbose())
            fprintf(stderr, "bship product plan: %lld result elements, %d candidates, first choice %.2f us, fastest (no. %d) %.2f us -> no. %d\n",
                    (long long)c_elements, found, first_ms * 1000.0f / 32.0f, fastest, best_ms * 1000.0f / 32.0f, best);
        (void)hipGetLastError();
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    pool_free_raw(scratch);
    return best;
}

// Column-major problem: D(m x n) = opA(A) opB(B), leading dimensions lda/ldb/ldc.
// tune: time the candidates on these operands instead of taking the heuristic's first choice.
// with_bias: the epilogue adds a vector of m elements to every column of D (the pointer is set per call).
int make_plan(GemmPlan& p, hipblasOperation_t opa, hipblasOperation_t opb, int64_t m, int64_t n,
              int64_t k, int64_t lda, int64_t ldb, int64_t ldc, bool with_bias, const TuneOperands* tune) {
    BSHIP_BLAS(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
    if (with_bias) {
        const uint32_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
        const int32_t bias_type = HIP_R_32F;
        BSHIP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)));
        BSHIP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)));
    }
    int32_t ta = static_cast<int32_t>(opa), tb = static_cast<int32_t>(opb);
    BSHIP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)));
    BSHIP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)));
    const bool na = (opa == HIPBLAS_OP_N), nb = (opb == HIPBLAS_OP_N);
    BSHIP_BLAS(hipblasLtMatrixLayoutCreate(&p.la, HIP_R_32F, na ? m : k, na ? k : m, lda));
    BSHIP_BLAS(hipblasLtMatrixLayoutCreate(&p.lb, HIP_R_32F, nb ? k : n, nb ? n : k, ldb));
    BSHIP_BLAS(hipblasLtMatrixLayoutCreate(&p.lc, HIP_R_32F, m, n, ldc));
    hipblasLtMatmulPreference_t pref = nullptr;
    BSHIP_BLAS(hipblasLtMatmulPreferenceCreate(&pref));
    uint64_t ws = kWorkspaceBytes;
    hipblasStatus_t s = hipblasLtMatmulPreferenceSetAttribute(
        pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
    constexpr int kCandidates = 24;
    hipblasLtMatmulHeuristicResult_t res[kCandidates];
    int found = 0;
    const int want = tune ? kCandidates : 1;
    if (s == HIPBLAS_STATUS_SUCCESS)
        s = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.la, p.lb, p.lc, p.lc, pref, want, res, &found);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (s != HIPBLAS_STATUS_SUCCESS) return blas_error(s, "hipblasLtMatmulAlgoGetHeuristic");
    if (found < 1)
        return set_error(BSHIP_ERR_BLAS,
                         "hipBLASLt has no float32 algorithm for m=%lld n=%lld k=%lld opA=%d opB=%d",
                         (long long)m, (long long)n, (long long)k, (int)opa, (int)opb);
    int best = 0;
    if (tune && found > 1) best = fastest_candidate(p, res, found, tune->a, tune->b, tune->bias, ldc * n);
    p.algo = res[best].algo;
    p.workspace = res[best].workspaceSize;
    return 0;
}

}  // namespace

void gemm_release() {
    std::lock_guard<std::mutex> lock(g_gemm_mutex);
    for (auto& kv : g_plans) destroy_plan(kv.second);
    g_plans.clear();
    if (g_workspace) { (void)hipFree(g_workspace); g_workspace = nullptr; }
    if (g_handle) { hipblasLtDestroy(g_handle); g_handle = nullptr; }
}

}  // namespace bship

using namespace bship;

static int gemm_impl(int transa, int transb, int64_t M, int64_t N, int64_t K, float alpha, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float beta, const float* bias, float* C,
                     int64_t ldc) {
    std::lock_guard<std::mutex> lock(g_gemm_mutex);
    if (!g_handle) BSHIP_BLAS(hipblasLtCreate(&g_handle));
    if (!g_workspace) {
        hipError_t e = hipMalloc(&g_workspace, kWorkspaceBytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            g_workspace = nullptr;
            return set_error(BSHIP_ERR_OUT_OF_MEMORY, "hipMalloc of the %zu-byte product workspace failed: %s",
                             kWorkspaceBytes, hipGetErrorString(e));
        }
    }
    // Row-major C(MxN) = op(A) op(B)  <=>  column-major C^T(NxM) = op(B)^T op(A)^T.
    // A row-major matrix read as column-major is its transpose, so the first
    // column-major operand is B with opB, the second is A with opA. A bias per column of the
    // row-major C is a bias per row of C^T, which is what the library's epilogue adds.
    const GemmKey key(transa != 0, transb != 0, M, N, K, lda, ldb, ldc, bias != nullptr);
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        GemmPlan plan;
        // thin and small enough that a few dozen trial runs cost milliseconds; not while a step is recorded
        const bool autotune = tune_mode() >= 1;
        const bool thin = (M <= 128 || N <= 128) && 2.0 * M * N * K <= 8e9 && M * N >= 1024;
        const TuneOperands operands{B, A, bias};
        int st = make_plan(plan, transb ? HIPBLAS_OP_T : HIPBLAS_OP_N, transa ? HIPBLAS_OP_T : HIPBLAS_OP_N,
                           N, M, K, ldb, lda, ldc, bias != nullptr,
                           autotune && thin && !graph_recording() ? &operands : nullptr);
        if (st != 0) { destroy_plan(plan); return st; }
        if (g_plans.size() >= kMaxPlans) {
            // drop the shape that has not been used for the longest time (launches already
            // enqueued keep no reference to a plan)
            auto oldest = g_plans.begin();
            for (auto jt = g_plans.begin(); jt != g_plans.end(); ++jt)
                if (jt->second.last_use < oldest->second.last_use) oldest = jt;
            destroy_plan(oldest->second);
            g_plans.erase(oldest);
        }
        it = g_plans.emplace(key, plan).first;
    }
    it->second.last_use = ++g_use_counter;
    const GemmPlan& p = it->second;
    if (bias)
        BSHIP_BLAS(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
    BSHIP_BLAS(hipblasLtMatmul(g_handle, p.desc, &alpha, B, p.la, A, p.lb, &beta, C, p.lc, C, p.lc,
                               &p.algo, g_workspace, kWorkspaceBytes, ctx().stream));
    return check_launch("gemm");
}

extern "C" int bship_gemm_f32(int transa, int transb, int64_t M, int64_t N, int64_t K, float alpha,
                              const float* A, int64_t lda, const float* B, int64_t ldb, float beta,
                              float* C, int64_t ldc) {
    BSHIP_REQUIRE_INIT_NO_FLUSH();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0 && K >= 0);
    if (M == 0 || N == 0) return 0;
    BSHIP_REQUIRE_PTR(C);
    BSHIP_REQUIRE_DIM(ldc >= N);
    if (K == 0) {
        BSHIP_FLUSH_PENDING();
        // empty inner dimension: C = beta * C
        if (beta == 1.0f) return 0;
        if (ldc != N) return set_error(BSHIP_ERR_UNSUPPORTED, "bship_gemm_f32: K == 0 needs a dense C");
        return beta == 0.0f ? bship_fill_f32(C, 0.0f, static_cast<size_t>(M * N))
                            : bship_scalar_f32(BSHIP_MULT_ST, beta, C, C, static_cast<size_t>(M * N));
    }
    BSHIP_REQUIRE_PTR(A);
    BSHIP_REQUIRE_PTR(B);
    BSHIP_REQUIRE_DIM(lda >= (transa ? M : K));
    BSHIP_REQUIRE_DIM(ldb >= (transb ? K : N));
    if (g_window_on.load(std::memory_order_relaxed) == 2 && window_takes())      // mode "stacked": products are held too
        return window_push(window::rec_gemm(transa != 0, transb != 0, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc));
    if (g_window_held.load(std::memory_order_relaxed) != 0 && !t_window_emitting) {
        // A layer's products lie between its elementwise calls (lstm_layer.py:121-145). The product goes
        // ahead of the operations the fusing window holds when it shares no operand with them that either
        // side writes; otherwise they are enqueued first.
        const int64_t a_rows = transa ? K : M, a_cols = transa ? M : K, b_rows = transb ? N : K, b_cols = transb ? K : N;
        const void* rd[3] = {A, B, C};
        const size_t rd_len[3] = {static_cast<size_t>((a_rows - 1) * lda + a_cols) * 4,
                                  static_cast<size_t>((b_rows - 1) * ldb + b_cols) * 4,
                                  static_cast<size_t>((M - 1) * ldc + N) * 4};
        const void* wr[1] = {C};
        int st = window_before_product(rd, rd_len, beta != 0.0f ? 3 : 2, wr, rd_len + 2, 1);
        if (st != 0) return st;
    }
    if (g_deferred_fill_count.load(std::memory_order_relaxed) != 0) {
        int st = flush_deferred_fills();
        if (st != 0) return st;
    }
    return gemm_impl(transa, transb, M, N, K, alpha, A, lda, B, ldb, beta, nullptr, C, ldc);
}

extern "C" int bship_gemm_bias_f32(int transa, int transb, int64_t M, int64_t N, int64_t K, const float* A,
                                   int64_t lda, const float* B, int64_t ldb, const float* bias, float* C,
                                   int64_t ldc) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0 && K >= 1);
    if (M == 0 || N == 0) return 0;
    BSHIP_REQUIRE_PTR(A);
    BSHIP_REQUIRE_PTR(B);
    BSHIP_REQUIRE_PTR(bias);
    BSHIP_REQUIRE_PTR(C);
    BSHIP_REQUIRE_DIM(ldc >= N);
    BSHIP_REQUIRE_DIM(lda >= (transa ? M : K));
    BSHIP_REQUIRE_DIM(ldb >= (transb ? K : N));
    return gemm_impl(transa, transb, M, N, K, 1.0f, A, lda, B, ldb, 0.0f, bias, C, ldc);
}
