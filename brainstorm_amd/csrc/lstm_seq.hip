// The forward recurrence of a peephole LSTM layer (lstm_layer.py:115-145) for ALL time steps in one
// persistent launch.
//
// Step by step through the library, a time step is one float32 product y[t-1] (B,H) x [Rz;Ri;Rf;Ro]^T
// (4H,H) and one elementwise kernel: for B = 100, H = 1000 the product alone takes 13.7 us, re-reads the
// 16 MB of recurrent weights from the L2s every step and is followed by a launch gap. Here the weights
// stay on chip for the whole sequence: a workgroup owns 4 hidden units, i.e. the 16 rows
// {z,i,f,o} x {4 units} of the stacked matrix (64 KB in LDS), and has a compute unit to itself. It computes
// the (B,16) slab of pre-activations of its units with float32 matrix-core instructions
// (v_mfma_f32_16x16x4f32), applies the cell update to its (B,4) elements, writes y[t] and the ten
// internals, and meets the other workgroups at one grid barrier per time step.
//
// Row sets: four wavefronts (the K quarters) handle up to 64 rows of the batch, as up to 4 row tiles of 16;
// a batch above 64 rows gets a second set of four wavefronts in the same workgroup (7 tiles are 4 + 3).
//
// The operand y[t-1] is kept TRANSPOSED (k-major, 128 columns of batch) in scratch buffers beside the
// layer's own y, one per time step, because the matrix-core operand layout gives neighbouring lanes
// neighbouring batch rows: v_mfma_f32_16x16x4f32 (A 16x4, B 4x16, D 16x16, one float of A and B and four of D per lane)
// takes A[l % 16][l / 16] and B[l / 16][l % 16] from lane l and returns D[4 * (l / 16) + r][l % 16], r = 0..3.
// Read from the (B,H) array, the 16 lanes of a group would touch 16 different rows with one load; read
// from the transposed copy, lane (m = l % 16, g = l / 16) loads the NT consecutive batch rows
// base + NT*m .. + NT-1 of row k of the copy, and component r of that load is its operand for row tile r,
// whose 16 rows are the batch rows base + NT*m' + r (a tile need not be contiguous). NT = 1..4 is the number
// of 16-row tiles the row set's rows need.
//
// Inside a row set wavefront w takes the K-quarter w of the inner dimension for all of the set's tiles; the
// four K-partial sums of an element meet in LDS and are added in a fixed order.
//
// The grid barrier: y[t] goes to the step's transposed buffer with write-through stores; every wavefront
// waits for its stores, the workgroup's first wavefront raises the workgroup's flag in device memory to the
// step number and polls all flags (four loads in flight). No cache is
// invalidated: a buffer is written once and read only afterwards, so no L1 or L2 can hold an older copy of
// its lines (only when the sequence needs more scratch than the limit are buffers reused, and then the
// compute unit's and the L2's lines are dropped at every barrier). The wait is bounded: after `spin_limit` polls a workgroup sets *failed and every workgroup
// exits at its next poll, so the kernel ends in any case; the host then reports the failure. All
// workgroups must be resident together: the host checks the occupancy the runtime reports against the
// grid before it launches.
#pragma clang fp contract(off)

#include <cstdlib>

#include <cerrno>
#include <mutex>

#include "buffer_loads.h"
#include "common.h"
#include "functors.h"
#include "lstm_cell.h"

namespace bship {

// The value of an environment variable that must be a whole number in [0, most]; `fallback` when it is
// unset, empty, not a number, followed by anything, or too large.
static unsigned long long env_number(const char* name, unsigned long long fallback, unsigned long long most) {
    const char* text = getenv(name);
    if (!text || !text[0]) return fallback;
    char* end = nullptr;
    errno = 0;
    const unsigned long long v = strtoull(text, &end, 10);
    if (errno != 0 || end == text || *end != 0 || text[0] == '-' || v > most) return fallback;
    return v;
}

constexpr int kSeqSetThreads = 256;               // the four wavefronts (K quarters) of one row set
constexpr int kSeqUnits = 4;                      // hidden units per workgroup
constexpr int kSeqCols = 4 * kSeqUnits;           // one 16-column tile: gates z, i, f, o of the units
constexpr int kSeqSetRows = 64;                   // batch rows per row set: up to 4 row tiles of 16
constexpr int kSeqMaxBatch = 2 * kSeqSetRows;     // two row sets; also the columns of the transposed operand
constexpr int kSeqMaxGroups = 256;                // workgroups (flags) at most

typedef float v4f __attribute__((ext_vector_type(4)));

struct LstmSeqArgs {
    float *Za, *Zb, *Ia, *Ib, *Fa, *Fb, *Oa, *Ob, *Ca, *Cb, *y;   // (T + 1, B, H) each; slab T is the context slot
    const float *R;                                               // (4H, H): [Rz; Ri; Rf; Ro]
    const float *pi, *pf, *po, *bz, *bi, *bf, *bo;                // (H,) each
    float* yT;             // nbuf (krows, 128) buffers: step t reads y[t-1] transposed from buffer t % nbuf
    int nbuf;              // T + 1 when that fits the scratch limit (no buffer is ever rewritten), else at least 2
    int reuse;             // nbuf < T + 1: buffers are rewritten, caches must drop their old lines at every barrier
    unsigned* flags;       // one per workgroup, zero on entry
    int* failed;           // zero on entry; 1 if a wait ran out
    int T, B, H, act;
    int base1;             // first batch row of row set 1 (set 0 starts at row 0)
    int nt0, nt1;          // row tiles of set 0 and set 1 (nt1 == 0: one set, 256 lanes)
    int kpitch;            // floats from one weight row to the next in LDS
    int kquarter;          // k values per wavefront (a multiple of 16)
    int krows;             // 4 * kquarter: rows of a transposed-operand buffer
    unsigned spin_limit;
};

// One wavefront's share of a time step's product: the NT row tiles of its row set (batch rows base + NT*m' + r)
// times the workgroup's 16 weight rows over the wavefront's K quarter, left in P[kq][batch row][column].
// No barrier inside: the two row sets of a workgroup run different instances.
template <int NT>
__device__ __forceinline__ void lstm_sequence_product(const LstmSeqArgs& a, const float* Rs, float* P,
                                                      __amdgpu_buffer_rsrc_t yprev, int base, int kq, int lane,
                                                      int k_begin, int nblocks, int rot) {
    const int m = lane & 15, g = lane >> 4;
    v4f acc[NT];
#pragma unroll
    for (int r = 0; r < NT; ++r) acc[r] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    // A k block is 16 wide. Lane (m, g) takes k = kb + 4g + j, j = 0..3: four weights with one LDS read,
    // and for each j its NT batch rows of row k of the transposed operand with one load (16 neighbouring
    // lanes read 64 * NT contiguous bytes).
    struct Block { Piece<NT> ya[4]; v4f rb; };
    auto load_block = [&](int ib, Block& blk) {
        int b = (ib < nblocks ? ib : nblocks - 1) + rot;           // past the end: the last block's weights (not used)
        if (b >= nblocks) b -= nblocks;
        const int k = k_begin + 16 * b + 4 * g;
        blk.rb = *reinterpret_cast<const v4f*>(Rs + m * a.kpitch + k);
        const int voff = ib < nblocks ? (k * kSeqMaxBatch + base + NT * m) * 4 : kBufferOob;
#pragma unroll
        for (int j = 0; j < 4; ++j) blk.ya[j] = load_piece<NT>(yprev, voff + j * kSeqMaxBatch * 4);
    };
    auto multiply = [&](const Block& blk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int r = 0; r < NT; ++r)
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(blk.ya[j].v[r], blk.rb[j], acc[r], 0, 0, 0);
        }
    };
    // With every compute unit of an XCD pulling the same operand out of one L2, a load takes about two
    // microseconds to come back and a block is multiplied in a seventh of that: loads run kSets - 1 blocks
    // ahead, in kSets register sets used in turn. Every load is issued unconditionally (one past the last
    // block reads beyond the buffer: zeros, no memory access), which lets the compiler wait for exactly the
    // set it needs and leave the younger ones in flight.
    if (nblocks > 0) {
        constexpr int kSets = NT == 4 ? 4 : (NT == 3 ? 5 : 8);    // what 256 registers per lane hold beside the cell state
        Block blk[kSets];
#pragma unroll
        for (int s = 0; s < kSets - 1; ++s) load_block(s, blk[s]);
        for (int ib = 0; ib < nblocks; ib += kSets) {
#pragma unroll
            for (int s = 0; s < kSets; ++s) {
                load_block(ib + s + kSets - 1, blk[(s + kSets - 1) % kSets]);
                if (ib + s < nblocks) multiply(blk[s]);
            }
        }
    }
    // lane (m, g) holds, of tile r, the rows m' = 4g + q (q = 0..3) of column m: batch row base + NT * m' + r
#pragma unroll
    for (int r = 0; r < NT; ++r) {
#pragma unroll
        for (int q = 0; q < 4; ++q) P[(kq * kSeqMaxBatch + base + NT * (4 * g + q) + r) * kSeqCols + m] = acc[r][q];
    }
}

// two wavefronts per SIMD at most: one workgroup per compute unit
__global__ __launch_bounds__(2 * kSeqSetThreads) void lstm_fwd_sequence_kernel(LstmSeqArgs a) {
    extern __shared__ float seq_lds[];
    float* Rs = seq_lds;                                                     // [16][kpitch]
    float* P = seq_lds + kSeqCols * a.kpitch;                                // [4][kSeqMaxBatch][16]
    __shared__ int s_go;
    const int tid = static_cast<int>(threadIdx.x);
    const int lane = tid & 63, wave = tid >> 6;
    const int kq = wave & 3, set = wave >> 2;
    const int H = a.H;
    const int ug = static_cast<int>(blockIdx.x);
    const int u0 = ug * kSeqUnits;
    const int64_t slab = static_cast<int64_t>(a.B) * H;
    const unsigned members = gridDim.x;

    // `between` runs after the workgroup has announced its arrival and before it looks for the others:
    // the place for stores nobody waits for.
    auto grid_barrier = [&](unsigned target, auto between) -> bool {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // this wavefront's write-through stores have reached memory
        __syncthreads();
        if (tid == 0) __hip_atomic_store(a.flags + ug, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        between();
        if (wave == 0) {
            int go = 1;
            unsigned spins = 0;
            for (;;) {
                // a limit of 0 polls gives up at once: the way to exercise this path from the host
                if (spins++ >= a.spin_limit || __hip_atomic_load(a.failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                    if (lane == 0) __hip_atomic_store(a.failed, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    go = 0;
                    break;
                }
                // the flags, four per lane, all four loads in flight together (a lane beyond the last
                // workgroup reads the last one's flag again)
                unsigned seen[kSeqMaxGroups / 64];
#pragma unroll
                for (int i = 0; i < kSeqMaxGroups / 64; ++i) {
                    const unsigned w = static_cast<unsigned>(lane) + 64u * i;
                    seen[i] = __hip_atomic_load(a.flags + (w < members ? w : members - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                bool here = true;
#pragma unroll
                for (int i = 0; i < kSeqMaxGroups / 64; ++i) here = here && seen[i] >= target;
                if (__all(here)) break;
            }
            // With a buffer per time step nobody has read the operand's lines before they were written, so no
            // cache holds a stale copy; with fewer buffers than steps this compute unit's and this L2's stale
            // lines are dropped here.
            if (a.reuse) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            if (lane == 0) s_go = go;
        }
        __syncthreads();
        return s_go != 0;                                         // the same for every lane of the workgroup
    };

    // this workgroup's 16 weight rows -> LDS (row c = gate * 4 + unit), zero beyond H and for missing units
    for (int c = 0; c < kSeqCols; ++c) {
        const int unit = u0 + (c & 3), gate = c >> 2;
        const float* src = a.R + (static_cast<int64_t>(gate) * H + unit) * H;
        for (int k = tid; k < a.kpitch; k += static_cast<int>(blockDim.x))
            Rs[c * a.kpitch + k] = (unit < H && k < H) ? src[k] : 0.0f;
    }
    // the element of the (B, 4) slab this lane updates, its previous cell state and its input products
    // (fetched a step ahead: they do not depend on other workgroups)
    const int eb = tid >> 2, eu = tid & 3;          // batch row, unit inside the workgroup
    const int ej = u0 + eu;
    const bool owns = eb < a.B && ej < H;
    float c_prev = 0.0f, p_i = 0.0f, p_f = 0.0f, p_o = 0.0f, b_z = 0.0f, b_i = 0.0f, b_f = 0.0f, b_o = 0.0f;
    float in_z = 0.0f, in_i = 0.0f, in_f = 0.0f, in_o = 0.0f;
    float* const yT0 = a.yT;                                     // buffer 0; the others follow it
    const int64_t yT_step = static_cast<int64_t>(a.krows) * kSeqMaxBatch;
    // what a load may touch of a buffer: the rows of real hidden units. Rows beyond them read zeros (the k
    // padding of the last block), so the buffers need no clearing: columns beyond the batch hold whatever the
    // pool block held, and those only reach rows of the product that nobody reads.
    const int yT_bytes = H * kSeqMaxBatch * static_cast<int>(sizeof(float));
    if (owns) {
        const int64_t e0 = static_cast<int64_t>(eb) * H + ej;
        c_prev = a.Ca[static_cast<int64_t>(a.T) * slab + e0];                                   // Ca[-1]
        p_i = a.pi[ej]; p_f = a.pf[ej]; p_o = a.po[ej];
        b_z = a.bz[ej]; b_i = a.bi[ej]; b_f = a.bf[ej]; b_o = a.bo[ej];
        in_z = a.Za[e0]; in_i = a.Ia[e0]; in_f = a.Fa[e0]; in_o = a.Oa[e0];
        // y[-1], transposed, is what step 0 multiplies
        __hip_atomic_store(yT0 + ej * kSeqMaxBatch + eb, a.y[static_cast<int64_t>(a.T) * slab + e0], __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!grid_barrier(1u, [] {})) return;

    const int nt = set == 0 ? a.nt0 : a.nt1;
    const int base = set == 0 ? 0 : a.base1;
    const int k_begin = kq * a.kquarter;
    const int k_limit = (H + 15) & ~15;
    const int k_end = k_begin + a.kquarter < k_limit ? k_begin + a.kquarter : k_limit;
    const int nblocks = k_end > k_begin ? (k_end - k_begin) / 16 : 0;
    // All workgroups of an XCD read the same y[t-1] out of the same L2 at the same time; if they also walked
    // it in the same order, every request of a moment would go to the same L2 channel. Each workgroup
    // therefore starts its k blocks at a different one (and wraps around).
    const int rot = nblocks > 0 ? static_cast<int>((blockIdx.x / 8u) % static_cast<unsigned>(nblocks)) : 0;
    // What a step leaves besides its operand for the next one (y[t] and the ten internals) is stored while
    // the workgroup waits at the barrier.
    LstmCell cell = {};
    int64_t e = 0;
    auto store_results = [&] {
        if (owns) {
            a.y[e] = cell.y;
            a.Za[e] = cell.za; a.Zb[e] = cell.zb; a.Ia[e] = cell.ia; a.Ib[e] = cell.ib; a.Fa[e] = cell.fa; a.Fb[e] = cell.fb;
            a.Ca[e] = cell.ca; a.Oa[e] = cell.oa; a.Ob[e] = cell.ob; a.Cb[e] = cell.cb;
        }
    };
    for (int t = 0; t < a.T; ++t) {
        e = static_cast<int64_t>(t) * slab + static_cast<int64_t>(eb) * H + ej;
        const __amdgpu_buffer_rsrc_t yprev = uniform_rsrc(yT0 + (t % a.nbuf) * yT_step, yT_bytes);
        switch (nt) {
            case 1: lstm_sequence_product<1>(a, Rs, P, yprev, base, kq, lane, k_begin, nblocks, rot); break;
            case 2: lstm_sequence_product<2>(a, Rs, P, yprev, base, kq, lane, k_begin, nblocks, rot); break;
            case 3: lstm_sequence_product<3>(a, Rs, P, yprev, base, kq, lane, k_begin, nblocks, rot); break;
            case 4: lstm_sequence_product<4>(a, Rs, P, yprev, base, kq, lane, k_begin, nblocks, rot); break;
            default: break;
        }
        __syncthreads();
        if (owns) {
            float rec[4];
#pragma unroll
            for (int gate = 0; gate < 4; ++gate) {
                const int col = gate * 4 + eu;
                const float p0 = P[(0 * kSeqMaxBatch + eb) * kSeqCols + col], p1 = P[(1 * kSeqMaxBatch + eb) * kSeqCols + col];
                const float p2 = P[(2 * kSeqMaxBatch + eb) * kSeqCols + col], p3 = P[(3 * kSeqMaxBatch + eb) * kSeqCols + col];
                rec[gate] = (p0 + p1) + (p2 + p3);
            }
            cell.za = in_z + rec[0];
            cell.ia = in_i + rec[1];
            cell.fa = in_f + rec[2];
            cell.oa = in_o + rec[3];
            if (t + 1 < a.T) { in_z = a.Za[e + slab]; in_i = a.Ia[e + slab]; in_f = a.Fa[e + slab]; in_o = a.Oa[e + slab]; }
            lstm_cell_forward(cell, a.act, c_prev, p_i, p_f, p_o, b_z, b_i, b_f, b_o);
            // the next step's operand first, written through to memory
            if (t + 1 < a.T)
                __hip_atomic_store(yT0 + ((t + 1) % a.nbuf) * yT_step + ej * kSeqMaxBatch + eb, cell.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            c_prev = cell.ca;
        }
        if (t + 1 == a.T) { store_results(); break; }              // nothing follows the last step
        if (!grid_barrier(static_cast<unsigned>(t) + 2u, store_results)) return;
    }
}

}  // namespace bship

using namespace bship;

extern "C" int bship_lstm_fwd_sequence_f32(int act, int64_t time_steps, int64_t batch, int64_t n, const float* R_all,
                                           float* Za, float* Zb, float* Ia, float* Ib, float* Fa, float* Fb,
                                           float* Oa, float* Ob, float* Ca, float* Cb, float* y, const float* pi,
                                           const float* pf, const float* po, const float* bz, const float* bi,
                                           const float* bf, const float* bo) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_EAGER();
    BSHIP_REQUIRE_DIM(time_steps >= 0 && batch >= 0 && n >= 0);
    if (act < 0 || act > 4) return set_error(BSHIP_ERR_BAD_OP, "%s: unknown activation %d", __func__, act);
    if (time_steps == 0 || batch == 0 || n == 0) return 0;
    const float* ins[] = {R_all, pi, pf, po, bz, bi, bf, bo};
    float* outs[] = {Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y};
    for (const float* p : ins) { BSHIP_REQUIRE_PTR(p); BSHIP_REQUIRE_F32_ALIGNED(p); }
    for (float* p : outs) { BSHIP_REQUIRE_PTR(p); BSHIP_REQUIRE_F32_ALIGNED(p); }
    const Context& c = ctx();
    const int64_t ugroups = ceil_div(n, kSeqUnits);
    if (n % 4 != 0 || batch > kSeqMaxBatch || ugroups > kSeqMaxGroups || time_steps > 0x3fffff)
        return set_error(BSHIP_ERR_UNSUPPORTED, "%s: needs n %% 4 == 0, batch <= %d and n <= %d; got batch %lld, n %lld",
                         __func__, kSeqMaxBatch, kSeqUnits * kSeqMaxGroups, static_cast<long long>(batch),
                         static_cast<long long>(n));
    LstmSeqArgs a;
    a.Za = Za; a.Zb = Zb; a.Ia = Ia; a.Ib = Ib; a.Fa = Fa; a.Fb = Fb; a.Oa = Oa; a.Ob = Ob; a.Ca = Ca; a.Cb = Cb; a.y = y;
    a.R = R_all; a.pi = pi; a.pf = pf; a.po = po; a.bz = bz; a.bi = bi; a.bf = bf; a.bo = bo;
    a.T = static_cast<int>(time_steps); a.B = static_cast<int>(batch); a.H = static_cast<int>(n); a.act = act;
    // row tiles: one set of up to 4, or two sets that share them as evenly as they divide
    const int tiles = static_cast<int>(ceil_div(batch, 16));
    a.nt0 = tiles <= 4 ? tiles : (tiles + 1) / 2;
    a.nt1 = tiles - a.nt0;
    a.base1 = 16 * a.nt0;
    const int sets = a.nt1 > 0 ? 2 : 1;
    const int k16 = (a.H + 15) & ~15;
    a.kquarter = ((k16 / 16 + 3) / 4) * 16;
    a.krows = 4 * a.kquarter;
    int kpitch = k16;                                  // covers every k a wavefront reads
    if ((kpitch / 4) % 2 == 0) kpitch += 4;            // an odd number of 16-byte units per row spreads the rows over the banks
    a.kpitch = kpitch;
    // BSHIP_GRID_BARRIER_SPINS: polls a workgroup spends at a barrier before it gives up. A value that is
    // not a whole number is ignored; 0 is the test hook that makes every barrier fail at once.
    a.spin_limit = static_cast<unsigned>(env_number("BSHIP_GRID_BARRIER_SPINS", 1u << 21, 0xffffffffull));
    const size_t lds = (static_cast<size_t>(kSeqCols) * kpitch + 4 * kSeqMaxBatch * kSeqCols) * sizeof(float);
    {
        static std::once_flag lds_once;
        static hipError_t lds_status = hipSuccess;
        std::call_once(lds_once, [] {
            lds_status = hipFuncSetAttribute(reinterpret_cast<const void*>(lstm_fwd_sequence_kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 1024);
        });
        BSHIP_HIP(lds_status);
    }
    // More than half of a compute unit's LDS, so that two workgroups never share one: a second one would
    // take matrix-core time from the first without shortening anybody's step.
    const size_t lds_ask = lds < 82 * 1024 ? 82 * 1024 : lds;
    const int64_t grid = ugroups;
    const int threads = sets * kSeqSetThreads;
    int per_cu = 0;
    if (lds_ask <= 159 * 1024)
        BSHIP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(lstm_fwd_sequence_kernel),
                                                               threads, lds_ask));
    if (static_cast<int64_t>(per_cu) * c.num_cus < grid)
        return set_error(BSHIP_ERR_UNSUPPORTED, "%s: n %d needs %lld workgroups with %zu bytes of LDS resident together; "
                         "the device holds %d per compute unit on %d compute units", __func__, a.H,
                         static_cast<long long>(grid), lds_ask, per_cu, c.num_cus);
    // the failure flag, 256 bytes on the flags of both groups (zero-filled), 4 KB on the transposed buffers:
    // one per time step and one for y[-1] if that stays below 256 MB, else as many as do (at least two)
    const size_t one = static_cast<size_t>(a.krows) * kSeqMaxBatch * sizeof(float);
    // BSHIP_LSTM_SEQ_SCRATCH_MB: default 256; small values force buffers to be reused (anything that is not a
    // whole number of at least 1 is ignored)
    size_t cap_mb = static_cast<size_t>(env_number("BSHIP_LSTM_SEQ_SCRATCH_MB", 256, 1u << 20));
    if (cap_mb < 1) cap_mb = 256;
    const size_t cap = cap_mb << 20;
    int64_t nbuf = time_steps + 1;
    if (static_cast<size_t>(nbuf) * one > cap) nbuf = static_cast<int64_t>(cap / one) < 2 ? 2 : static_cast<int64_t>(cap / one);
    a.nbuf = static_cast<int>(nbuf);
    a.reuse = nbuf < time_steps + 1 ? 1 : 0;
    const size_t yt_bytes = static_cast<size_t>(nbuf) * one;
    void* sync = nullptr;
    int st = pool_alloc_raw(4096 + yt_bytes, &sync);
    if (st != 0) return st;
    st = launch_fill(static_cast<float*>(sync), 0.0f, 1024);       // the flags; the operand buffers need no clearing
    if (st != 0) { pool_free_raw(sync); return st; }
    a.failed = static_cast<int*>(sync);
    a.flags = reinterpret_cast<unsigned*>(static_cast<char*>(sync) + 256);
    a.yT = reinterpret_cast<float*>(static_cast<char*>(sync) + 4096);
    hipLaunchKernelGGL(lstm_fwd_sequence_kernel, dim3(static_cast<unsigned>(grid)), dim3(threads), lds_ask,
                       c.stream, a);
    st = check_launch("lstm_forward_sequence");
    int failed = 0;
    if (st == 0) st = bship_d2h(&failed, a.failed, sizeof(int));     // waits for the kernel
    pool_free_raw(sync);
    if (st != 0) return st;
    if (failed)
        return set_error(BSHIP_ERR_TIMEOUT, "%s: the workgroups did not all meet at a time step's barrier within %u "
                         "polls (the device was shared with other work?); the layer's buffers hold an unfinished pass",
                         __func__, a.spin_limit);
    return 0;
}
