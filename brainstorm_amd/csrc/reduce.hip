// Reductions: sum_t over axis 0, axis 1 or everything, the fused one-pass row
// softmax, and the is_fully_finite check. Each input element is read from HBM
// exactly once. Results are deterministic: partial sums are combined in a
// fixed order (no floating-point atomics).
#pragma clang fp contract(off)

#include "common.h"
#include "window.h"
#include "colsum.h"

namespace bship {

// ============================ sum over axis 1 ==============================
// Row sums. THREADS lanes cooperate on one row (64 = one wavefront, 4 rows per
// workgroup; 256 = the whole workgroup). Lanes stride over the row, W floats
// per access; a row tail that does not fill W floats is added scalar-wise.
template <int W, bool AL, int THREADS>
__global__ __launch_bounds__(kBlock) void rowsum_kernel(const float* __restrict__ a,
                                                        float* __restrict__ out, int64_t M,
                                                        int64_t N, int64_t ld) {
    constexpr int ROWS = kBlock / THREADS;
    typedef typename VecT<W>::type R;
    __shared__ float lds[kBlock / kWave];
    const int t = threadIdx.x % THREADS;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * ROWS + threadIdx.x / THREADS;
    float total = 0.0f;
    if (row < M) {
        const int64_t NW = N / W;
        const float* p = a + row * ld;
        R acc0 = vzero<R>(), acc1 = vzero<R>(), acc2 = vzero<R>(), acc3 = vzero<R>();
        int64_t i = t;
        for (; i + 3 * THREADS < NW; i += 4 * THREADS) {
            R x0 = vload<W, AL>(p + i * W);
            R x1 = vload<W, AL>(p + (i + THREADS) * W);
            R x2 = vload<W, AL>(p + (i + 2 * THREADS) * W);
            R x3 = vload<W, AL>(p + (i + 3 * THREADS) * W);
            acc0 += x0; acc1 += x1; acc2 += x2; acc3 += x3;
        }
        for (; i < NW; i += THREADS) acc0 += vload<W, AL>(p + i * W);
        total = hsum((acc0 + acc1) + (acc2 + acc3));
        for (int64_t j = NW * W + t; j < N; j += THREADS) total += p[j];
    }
    total = wave_sum(total);
    if (THREADS == kWave) {
        if (t == 0 && row < M) out[row] = total;
    } else {
        const int wv = threadIdx.x / kWave;
        if ((threadIdx.x & (kWave - 1)) == 0) lds[wv] = total;
        __syncthreads();
        if (threadIdx.x == 0 && row < M) out[row] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    }
}

// One thread per row, for very short rows.
__global__ __launch_bounds__(kBlock) void rowsum_small_kernel(const float* __restrict__ a,
                                                              float* __restrict__ out, int64_t M,
                                                              int64_t N, int64_t ld) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (row >= M) return;
    float s = 0.0f;
    for (int64_t j = 0; j < N; ++j) s += a[row * ld + j];
    out[row] = s;
}

template <int THREADS>
static void launch_rowsum_kernel(bool vec, bool al, dim3 grid, const float* a, float* out,
                                 int64_t M, int64_t N, int64_t ld) {
    hipStream_t s = ctx().stream;
    if (vec && al) hipLaunchKernelGGL((rowsum_kernel<4, true, THREADS>), grid, dim3(kBlock), 0, s, a, out, M, N, ld);
    else if (vec)  hipLaunchKernelGGL((rowsum_kernel<4, false, THREADS>), grid, dim3(kBlock), 0, s, a, out, M, N, ld);
    else           hipLaunchKernelGGL((rowsum_kernel<1, false, THREADS>), grid, dim3(kBlock), 0, s, a, out, M, N, ld);
}

// ld: elements from one row of a to the next (N for a dense matrix)
static int launch_rowsum(const float* a, float* out, int64_t M, int64_t N, int64_t ld) {
    if (N <= 16) {
        hipLaunchKernelGGL(rowsum_small_kernel, dim3(static_cast<unsigned>(ceil_div(M, kBlock))),
                           dim3(kBlock), 0, ctx().stream, a, out, M, N, ld);
        return check_launch("sum_t(axis=1) small");
    }
    // every row starts on a 16-byte boundary only if the pitch is a whole number of vectors and the base does
    const bool vec = (N % 4 == 0);
    const bool al = aligned16(a) && ld % 4 == 0;
    if (N <= 2048)
        launch_rowsum_kernel<kWave>(vec, al, dim3(static_cast<unsigned>(ceil_div(M, kBlock / kWave))), a, out, M, N, ld);
    else
        launch_rowsum_kernel<kBlock>(vec, al, dim3(static_cast<unsigned>(M)), a, out, M, N, ld);
    return check_launch("sum_t(axis=1)");
}

// ============================== sum of all =================================
// Stage 1: `chunks` workgroups each sum one contiguous chunk of `len` floats (the
// last chunk may be shorter) into partial[chunk]; stage 2: one workgroup adds
// the partials in chunk order. (A single-launch variant in which the last
// workgroup to finish adds the partials was measured 4-10x slower on MI355X:
// the device-scope release fence every workgroup needs writes back the L2.)
template <bool AL>
__global__ __launch_bounds__(kBlock) void sumchunk_kernel(const float* __restrict__ a,
                                                          float* __restrict__ partial, size_t n,
                                                          size_t len) {
    __shared__ float lds[kBlock / kWave];
    const size_t begin = static_cast<size_t>(blockIdx.x) * len;
    const size_t end = begin + len < n ? begin + len : n;
    const size_t nvec = (end - begin) / 4;
    const float* p = a + begin;
    f4 acc0 = vzero<f4>(), acc1 = vzero<f4>(), acc2 = vzero<f4>(), acc3 = vzero<f4>();
    size_t i = threadIdx.x;
    for (; i + 3 * kBlock < nvec; i += 4 * kBlock) {
        f4 x0 = vload<4, AL>(p + i * 4);
        f4 x1 = vload<4, AL>(p + (i + kBlock) * 4);
        f4 x2 = vload<4, AL>(p + (i + 2 * kBlock) * 4);
        f4 x3 = vload<4, AL>(p + (i + 3 * kBlock) * 4);
        acc0 += x0; acc1 += x1; acc2 += x2; acc3 += x3;
    }
    for (; i < nvec; i += kBlock) acc0 += vload<4, AL>(p + i * 4);
    float total = hsum((acc0 + acc1) + (acc2 + acc3));
    for (size_t j = begin + nvec * 4 + threadIdx.x; j < end; j += kBlock) total += a[j];
    total = wave_sum(total);
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = total;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
}

static int launch_sumall(const float* a, float* out, int64_t n, PartialsBuffer ws = PartialsBuffer()) {
    const Context& c = ctx();
    const int64_t min_chunk = 16384;
    int64_t chunks = static_cast<int64_t>(c.num_cus) * 8;
    if (chunks > n / min_chunk) chunks = n / min_chunk;
    if (chunks < 1) chunks = 1;
    // chunk length: a multiple of 1024 floats so that every chunk start keeps the base alignment
    const int64_t len = ceil_div(ceil_div(n, chunks), 1024) * 1024;
    chunks = ceil_div(n, len);
    float* dst = out;
    float* partial = nullptr;
    if (chunks > 1 && ws.ptr) {
        if (static_cast<size_t>(chunks) > ws.floats)
            return set_error(BSHIP_ERR_BAD_DIMENSION,
                             "sum of %lld elements needs %lld floats of partial sums, the buffer given holds %zu",
                             static_cast<long long>(n), static_cast<long long>(chunks), ws.floats);
        dst = ws.ptr;
    } else if (chunks > 1) {
        void* p = nullptr;
        int st = pool_alloc_raw(static_cast<size_t>(chunks) * sizeof(float), &p);
        if (st != 0) return st;
        partial = static_cast<float*>(p);
        dst = partial;
    }
    const dim3 grid(static_cast<unsigned>(chunks));
    if (aligned16(a))
        hipLaunchKernelGGL(sumchunk_kernel<true>, grid, dim3(kBlock), 0, c.stream, a, dst,
                           static_cast<size_t>(n), static_cast<size_t>(len));
    else
        hipLaunchKernelGGL(sumchunk_kernel<false>, grid, dim3(kBlock), 0, c.stream, a, dst,
                           static_cast<size_t>(n), static_cast<size_t>(len));
    int st = check_launch("sum_t(axis=None) stage 1");
    if (dst != out) {
        if (st == 0) {
            launch_rowsum_kernel<kBlock>(false, false, dim3(1), dst, out, 1, chunks, chunks);
            st = check_launch("sum_t(axis=None) stage 2");
        }
        if (partial) pool_free_raw(partial);
    }
    return st;
}

// ================================ softmax ==================================
// exp(x) for x <= 0 (softmax exponents are differences to the row maximum):
// x*log2(e) split into an integer k and a remainder |r| <= 1/2 with the low part
// of log2(e) carried along, 2^r from the hardware exp2 (1 ulp), scaled by 2^k.
// About 2 ulp, a quarter of the instructions of the full-range expf; the softmax
// bar is 1e-5 relative.
__device__ __forceinline__ float exp_nonpositive(float x) {
    const float kLog2eHi = 1.44269502162933349609375f;      // float32(log2 e)
    const float kLog2eLo = 1.925963033500011e-8f;           // log2 e - float32(log2 e)
    const float k = rintf(x * kLog2eHi);
    float r = fmaf(x, kLog2eHi, -k);
    r = fmaf(x, kLog2eLo, r);
    const float e = ldexpf(__builtin_amdgcn_exp2f(r), static_cast<int>(k));
    return x < -104.0f ? 0.0f : e;                          // below 2^-150 (and -inf): zero
}

// One pass over HBM: THREADS lanes hold a whole row in registers (PER accesses
// of W floats each), reduce max and sum across the lanes, then write e/sum.
// THREADS is a wavefront (BLOCK/64 rows per workgroup) or the whole workgroup.
// Long rows take workgroups of 1024 lanes: measured on MI355X at 16384 columns,
// 4 vectors per lane x 1024 lanes reach 0.74 of peak where 16 x 256 reach 0.66.
// out = exp(m - rowmax) / sum(exp(m - rowmax))      (numpy 292-295)
// The launcher guarantees N % W == 0 and N / W <= THREADS * PER.
template <int W, bool AL, int BLOCK, int THREADS, int PER>
__global__ __launch_bounds__(BLOCK) void softmax_reg_kernel(const float* m, float* out, int64_t M,
                                                            int64_t N, int64_t ldm, int64_t ldo, unsigned chunk, bool through) {
    constexpr int ROWS = BLOCK / THREADS;
    constexpr int WAVES = BLOCK / kWave;
    typedef typename VecT<W>::type R;
    __shared__ float lds[2][WAVES];
    const int t = threadIdx.x % THREADS;
    // chunk > 1: the eight workgroups that the dispatcher deals to the eight XCDs in turn take rows
    // `chunk` apart, so that each XCD works on runs of `chunk` adjacent rows (see launch_softmax)
    unsigned bid = blockIdx.x;
    if (chunk > 1) {
        const unsigned full = gridDim.x / (8 * chunk) * (8 * chunk);
        if (bid < full) bid = (bid % 8) * chunk + (bid / 8) % chunk + (bid / (8 * chunk)) * (8 * chunk);
    }
    const int64_t row = static_cast<int64_t>(bid) * ROWS + threadIdx.x / THREADS;
    const bool live = row < M;
    const int64_t NW = N / W;
    const float* p = m + (live ? row : 0) * ldm;       // ldm, ldo: elements from one row to the next
    float* q = out + (live ? row : 0) * ldo;
    // All loads are issued before anything depends on one of them: lanes beyond the row's
    // end read element 0 instead (always valid) and are replaced by -inf afterwards, so
    // the loads sit in no branch and the wavefront keeps PER of them in flight.
    R x[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int64_t i = t + static_cast<int64_t>(k) * THREADS;
        x[k] = vload<W, AL>(p + ((live && i < NW) ? i : 0) * W);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int64_t i = t + static_cast<int64_t>(k) * THREADS;
        if (!(live && i < NW)) x[k] = vzero<R>() - INFINITY;
        mx = fmaxf(mx, hmax(x[k]));
    }
    mx = wave_max(mx);
    if (THREADS > kWave) {
        if ((threadIdx.x & (kWave - 1)) == 0) lds[0][threadIdx.x / kWave] = mx;
        __syncthreads();
        mx = lds[0][0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) mx = fmaxf(mx, lds[0][w]);
    }
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int64_t i = t + static_cast<int64_t>(k) * THREADS;
        if constexpr (W == 4) {
#pragma unroll
            for (int j = 0; j < 4; ++j) x[k][j] = exp_nonpositive(x[k][j] - mx);
        } else {
            x[k] = exp_nonpositive(x[k] - mx);
        }
        if (live && i < NW) sum += hsum(x[k]);       // padding lanes hold exp(-inf - mx), not counted
    }
    sum = wave_sum(sum);
    if (THREADS > kWave) {
        if ((threadIdx.x & (kWave - 1)) == 0) lds[1][threadIdx.x / kWave] = sum;
        __syncthreads();
        sum = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w += 4) sum += (lds[1][w] + lds[1][w + 1]) + (lds[1][w + 2] + lds[1][w + 3]);
    }
    const float inv = 1.0f / sum;        // one division per lane; e * inv is within 1 ulp of e / sum
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int64_t i = t + static_cast<int64_t>(k) * THREADS;
        if (live && i < NW) {
            R r;
            if constexpr (W == 4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) r[j] = x[k][j] * inv;
            } else {
                r = x[k] * inv;
            }
            vstore<W, AL>(q + i * W, r, through);
        }
    }
}

// Rows too long for registers: a workgroup per row, three sweeps (max, sum of
// exponentials, normalise); the second and third sweeps mostly hit the caches.
__global__ __launch_bounds__(kBlock) void softmax_long_kernel(const float* m, float* out, int64_t M,
                                                              int64_t N, int64_t ldm, int64_t ldo) {
    __shared__ float lds[kBlock / kWave];
    const int wv = threadIdx.x / kWave;
    const int64_t row = blockIdx.x;
    const float* p = m + row * ldm;
    float* q = out + row * ldo;
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < N; i += kBlock) mx = fmaxf(mx, p[i]);
    mx = wave_max(mx);
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wv] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
    __syncthreads();
    float sum = 0.0f;
    for (int64_t i = threadIdx.x; i < N; i += kBlock) sum += expf(p[i] - mx);
    sum = wave_sum(sum);
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wv] = sum;
    __syncthreads();
    sum = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    for (int64_t i = threadIdx.x; i < N; i += kBlock) q[i] = expf(p[i] - mx) / sum;
}

template <int W, bool AL, int BLOCK, int THREADS>
static void launch_softmax_per(int per, dim3 grid, const float* m, float* out, int64_t M, int64_t N, int64_t ldm,
                               int64_t ldo, unsigned chunk) {
    const bool through = store_through(static_cast<size_t>(M) * static_cast<size_t>(N));
    hipStream_t s = ctx().stream;
    const dim3 b(BLOCK);
    switch (per) {
        case 1:  hipLaunchKernelGGL((softmax_reg_kernel<W, AL, BLOCK, THREADS, 1>), grid, b, 0, s, m, out, M, N, ldm, ldo, chunk, through); break;
        case 2:  hipLaunchKernelGGL((softmax_reg_kernel<W, AL, BLOCK, THREADS, 2>), grid, b, 0, s, m, out, M, N, ldm, ldo, chunk, through); break;
        case 4:  hipLaunchKernelGGL((softmax_reg_kernel<W, AL, BLOCK, THREADS, 4>), grid, b, 0, s, m, out, M, N, ldm, ldo, chunk, through); break;
        case 8:  hipLaunchKernelGGL((softmax_reg_kernel<W, AL, BLOCK, THREADS, 8>), grid, b, 0, s, m, out, M, N, ldm, ldo, chunk, through); break;
        default: hipLaunchKernelGGL((softmax_reg_kernel<W, AL, BLOCK, THREADS, 16>), grid, b, 0, s, m, out, M, N, ldm, ldo, chunk, through); break;
    }
}

template <int BLOCK, int THREADS>
static void launch_softmax_threads(bool vec, bool al, int per, dim3 grid, const float* m, float* out,
                                   int64_t M, int64_t N, int64_t ldm, int64_t ldo, unsigned chunk = 0) {
    if (vec && al) launch_softmax_per<4, true, BLOCK, THREADS>(per, grid, m, out, M, N, ldm, ldo, chunk);
    else if (vec)  launch_softmax_per<4, false, BLOCK, THREADS>(per, grid, m, out, M, N, ldm, ldo, chunk);
    else           launch_softmax_per<1, false, BLOCK, THREADS>(per, grid, m, out, M, N, ldm, ldo, chunk);
}

constexpr int kWideBlock = 1024;
// Rows of up to this many accesses per lane are held by 256 lanes (8 workgroups fit a compute unit and
// overlap each other's load, arithmetic and store phases); measured at 8192 columns: 8 accesses x 256
// lanes reach 0.78 of peak, 2 x 1024 lanes 0.76. At 16384 columns 16 x 256 lanes fall to 0.67 against
// 0.70-0.72 for 4 x 1024, so longer rows take the wide workgroups.
#ifndef BSHIP_SM_NARROW_MAX
#define BSHIP_SM_NARROW_MAX 8
#endif

static int launch_softmax(const float* m, float* out, int64_t M, int64_t N, int64_t ldm, int64_t ldo) {
    const bool vec = (N % 4 == 0);
    const bool al = aligned16(m) && aligned16(out) && ldm % 4 == 0 && ldo % 4 == 0;
    const int64_t NW = vec ? N / 4 : N;
    // smallest power-of-two number of accesses per lane that covers the row
    auto per_for = [&](int threads) {
        int per = 1;
        while (per < 16 && static_cast<int64_t>(per) * threads < NW) per *= 2;
        return per;
    };
    if (NW <= static_cast<int64_t>(kWave) * 16) {
        // a wavefront per row, 4 rows per workgroup
        launch_softmax_threads<kBlock, kWave>(vec, al, per_for(kWave),
                                              dim3(static_cast<unsigned>(ceil_div(M, kBlock / kWave))), m, out, M, N, ldm, ldo);
    } else if (NW <= static_cast<int64_t>(kBlock) * BSHIP_SM_NARROW_MAX) {
        launch_softmax_threads<kBlock, kBlock>(vec, al, per_for(kBlock), dim3(static_cast<unsigned>(M)), m, out, M, N, ldm, ldo);
    } else if (NW <= static_cast<int64_t>(kWideBlock) * 16) {
        // Rows a multiple of 64 KiB apart: with one row per workgroup in index order, an XCD (every
        // eighth workgroup) would only ever see addresses that agree in bits 16-18, which costs 4-5 % at
        // 16384 x 16384 (0.71 -> 0.74 of peak with runs of 512 KiB per XCD; other pitches lose with runs).
        unsigned chunk = 0;
        if ((ldm * 4) % 65536 == 0 && (ldo * 4) % 65536 == 0) {
            chunk = static_cast<unsigned>(std::max<int64_t>(1, static_cast<int64_t>(ctx().softmax_run_bytes) / (ldm * 4)));
        }
        launch_softmax_threads<kWideBlock, kWideBlock>(vec, al, per_for(kWideBlock),
                                                       dim3(static_cast<unsigned>(M)), m, out, M, N, ldm, ldo, chunk);
    } else {
        hipLaunchKernelGGL(softmax_long_kernel, dim3(static_cast<unsigned>(M)), dim3(kBlock), 0,
                           ctx().stream, m, out, M, N, ldm, ldo);
    }
    return check_launch("softmax_m");
}

// ============================== is finite ==================================
__global__ __launch_bounds__(kBlock) void nonfinite_kernel(const float* __restrict__ a, size_t n,
                                                           int* __restrict__ flag) {
    bool bad = false;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * kBlock) {
        const uint32_t bits = __float_as_uint(a[i]);
        bad |= ((bits & 0x7f800000u) == 0x7f800000u);
    }
    if (bad) *flag = 1;    // every writer stores the same value
}

// ===================== partial sums without the pool ======================
// bship_sum_noalloc_f32 keeps the partial sums of its first stage here instead of in a pool
// block. 1 MiB per device, held until the process ends. In host code the array's name is only
// a stand-in for the symbol: the device address is looked up once per device
// (reduce_scratch_init) and every launch gets that pointer.
constexpr size_t kScratchFloats = size_t(1) << 18;
static __device__ __align__(256) float scratch[kScratchFloats];
constexpr int kMaxScratchDevices = 64;
static float* g_scratch_ptr[kMaxScratchDevices] = {nullptr};

// Called by bship_init with `device` current.
int reduce_scratch_init(int device) {
    if (device < 0 || device >= kMaxScratchDevices)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "device %d: no static partial-sum buffer beyond device %d",
                         device, kMaxScratchDevices - 1);
    if (g_scratch_ptr[device]) return 0;
    void* p = nullptr;
    int st = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(partial-sum buffer)");
    if (st != 0) return st;
    g_scratch_ptr[device] = static_cast<float*>(p);
    return 0;
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_sum_noalloc_f32(const float* a, float* out, int64_t M, int64_t N, int axis) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    BSHIP_REQUIRE_DIM(axis == 0 || axis == 1 || axis == -1);
    const int64_t out_n = axis == 0 ? N : (axis == 1 ? M : 1);
    if (out_n == 0) return 0;
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    if (M == 0 || N == 0) return launch_fill(out, 0.0f, static_cast<size_t>(out_n));  // empty sum
    BSHIP_REQUIRE_PTR(a);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    BSHIP_REQUIRE_DIM(a != out);
    BSHIP_REQUIRE_DIM(M <= 0x7fffffff);
    const int device = ctx().device;
    float* ws = device >= 0 && device < kMaxScratchDevices ? g_scratch_ptr[device] : nullptr;
    if (!ws) return set_error(BSHIP_ERR_NOT_INITIALIZED, "%s: no partial-sum buffer on device %d", __func__, device);
    const PartialsBuffer buf{ws, kScratchFloats};
    if (axis == 0) return M == 1 ? bship_d2d(out, a, static_cast<size_t>(N) * 4) : launch_colsum(PlainSrc{a}, out, M, N, N, buf);
    if (axis == 1) return N == 1 ? bship_d2d(out, a, static_cast<size_t>(M) * 4) : launch_rowsum(a, out, M, N, N);
    return launch_sumall(a, out, M * N, buf);
}

int bship_sum_f32(const float* a, float* out, int64_t M, int64_t N, int axis) {
    // column sums are part of the batch normalisation sequences: a dense sum goes through the fusing window
    if (window_takes() && M >= 1 && N >= 1 && M <= 0x7fffffff && (axis == 0 || axis == 1 || axis == -1) && a && out &&
        a != out && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(out)) & 3u) == 0) {
        BSHIP_REQUIRE_INIT_NO_FLUSH();
        return window_push(window::rec_sum(a, out, M, N, axis));
    }
    return bship_sum_pitched_f32(a, N, out, M, N, axis);       // reports what is wrong with the arguments, too
}

int bship_sum_pitched_f32(const float* a, int64_t ld_a, float* out, int64_t M, int64_t N, int axis) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    BSHIP_REQUIRE_DIM(ld_a >= N);
    BSHIP_REQUIRE_DIM(axis == 0 || axis == 1 || axis == -1);
    const int64_t out_n = axis == 0 ? N : (axis == 1 ? M : 1);
    if (out_n == 0) return 0;
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    if (M == 0 || N == 0) return launch_fill(out, 0.0f, static_cast<size_t>(out_n));  // empty sum
    BSHIP_REQUIRE_PTR(a);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    BSHIP_REQUIRE_DIM(a != out);
    BSHIP_REQUIRE_DIM(M <= 0x7fffffff);
    if (axis == 0) return M == 1 ? bship_d2d(out, a, static_cast<size_t>(N) * 4) : launch_colsum(PlainSrc{a}, out, M, N, ld_a);
    if (axis == 1) return N == 1 && ld_a == 1 ? bship_d2d(out, a, static_cast<size_t>(M) * 4) : launch_rowsum(a, out, M, N, ld_a);
    if (ld_a == N || M == 1) return launch_sumall(a, out, M * N);
    // everything, row-pitched: row sums, then their sum
    void* rows = nullptr;
    int st = pool_alloc_raw(static_cast<size_t>(M) * sizeof(float), &rows);
    if (st != 0) return st;
    st = launch_rowsum(a, static_cast<float*>(rows), M, N, ld_a);
    if (st == 0) st = launch_sumall(static_cast<const float*>(rows), out, M);
    pool_free_raw(rows);
    return st;
}

int bship_softmax_rows_f32(const float* m, float* out, int64_t M, int64_t N) {
    // the first call of the softmax cross-entropy layer's forward sequence: through the fusing window
    if (window_takes() && M >= 1 && N >= 1 && M <= 0x7fffffff && m && out &&
        ((reinterpret_cast<uintptr_t>(m) | reinterpret_cast<uintptr_t>(out)) & 3u) == 0) {
        BSHIP_REQUIRE_INIT_NO_FLUSH();
        return window_push(window::rec_softmax(m, out, M, N));
    }
    return bship_softmax_rows_pitched_f32(m, N, out, N, M, N);
}

int bship_softmax_rows_pitched_f32(const float* m, int64_t ld_m, float* out, int64_t ld_out, int64_t M, int64_t N) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    BSHIP_REQUIRE_DIM(ld_m >= N && ld_out >= N);
    if (M == 0 || N == 0) return 0;
    BSHIP_REQUIRE_PTR(m);
    BSHIP_REQUIRE_PTR(out);
    BSHIP_REQUIRE_F32_ALIGNED(m);
    BSHIP_REQUIRE_F32_ALIGNED(out);
    BSHIP_REQUIRE_DIM(M <= 0x7fffffff);
    return launch_softmax(m, out, M, N, ld_m, ld_out);
}

int bship_isfinite_f32(const float* a, size_t n, int* result_host) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_PTR(result_host);
    BSHIP_REQUIRE_EAGER();
    *result_host = 1;
    if (n == 0) return 0;
    BSHIP_REQUIRE_PTR(a);
    BSHIP_REQUIRE_F32_ALIGNED(a);
    void* p = nullptr;
    int st = pool_alloc_raw(sizeof(int), &p);
    if (st == 0) st = launch_fill(static_cast<float*>(p), 0.0f, 1);     // the flag starts at zero
    if (st != 0) { pool_free_raw(p); return st; }
    hipLaunchKernelGGL(nonfinite_kernel,
                       dim3(stream_grid(ceil_div(static_cast<int64_t>(n), kBlock * 4))),
                       dim3(kBlock), 0, ctx().stream, a, n, static_cast<int*>(p));
    st = check_launch("is_fully_finite");
    int flag = 0;
    if (st == 0) st = bship_d2h(&flag, p, sizeof(int));
    pool_free_raw(p);
    if (st == 0) *result_host = flag ? 0 : 1;
    return st;
}

}  // extern "C"
