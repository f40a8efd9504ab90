// Fused layer-level kernels: optional entry points that do in one launch what a
// brainstorm layer does with a dozen handler calls per time step. They are an
// extension, not part of the reference's handler interface; the primitive
// operations remain the default. Each kernel chains the very same per-element
// functors (functors.h) in the order the layer issues the primitive calls, so
// its results are bit-identical to the unfused sequence.
#pragma clang fp contract(off)

#include "colsum.h"
#include "common.h"
#include "window.h"
#include "functors.h"
#include "lstm_cell.h"

namespace bship {

// act_func_deriv[...](x, y, dy, dx) (base_handler.py:65-71); 'linear' copies dy
__device__ __forceinline__ float act_backward(int act, float y, float dy) {
    switch (act) {
        case kActSigmoid: return SigmoidDerivOp{}.apply(y, dy, 0.0f);
        case kActTanh:    return TanhDerivOp{}.apply(y, dy, 0.0f);
        case kActRel:     return RelDerivOp{}.apply(y, dy, 0.0f);
        case kActEl:      return ElDerivOp{}.apply(y, dy, 0.0f);
        default:          return dy;
    }
}

struct LstmFwdArgs {
    float *Za, *Zb, *Ia, *Ib, *Fa, *Fb, *Oa, *Ob, *Ca, *Cb, *y;
    const float *Ca_prev, *pi, *pf, *po, *bz, *bi, *bf, *bo;
    const float* rec;   // PACKED only: (batch, 4n) = y[t-1] [Rz;Ri;Rf;Ro]^T, columns [z|i|f|o]
};

// The elementwise part of one LSTM forward time step (lstm_layer.py:117-145),
// after the four recurrent products have been accumulated into Za, Ia, Fa, Oa:
//   add_mv(Za, bz); Zb = act(Za)
//   mult_add_mv(Ca_prev, pi, Ia); add_mv(Ia, bi); Ib = sigmoid(Ia)
//   mult_add_mv(Ca_prev, pf, Fa); add_mv(Fa, bf); Fb = sigmoid(Fa)
//   Ca = Ib * Zb; mult_add_tt(Fb, Ca_prev, Ca)
//   mult_add_mv(Ca, po, Oa); add_mv(Oa, bo); Ob = sigmoid(Oa)
//   Cb = act(Ca); y = Ob * Cb
//
// PACKED: the four recurrent products arrive as one (batch, 4n) matrix instead of
// having been accumulated into Za, Ia, Fa, Oa; they are added first, which is what
// the accumulating product does with its finished dot products.
// Streaming accesses of the step kernels: what a time step reads and writes once should not push
// the recurrent matrices, which the next step's product reads again, out of the L2 caches.
__device__ __forceinline__ float ldg(const float* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void stg(float* p, float v) { __builtin_nontemporal_store(v, p); }

template <bool PACKED>
__global__ __launch_bounds__(kBlock) void lstm_fwd_step_kernel(LstmFwdArgs a, int act, int64_t total,
                                                               unsigned n) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const unsigned j = static_cast<unsigned>(e % n);       // column: index into the (1,n) parameters
    const float c_prev = ldg(a.Ca_prev + e);
    float za = ldg(a.Za + e), ia = ldg(a.Ia + e), fa = ldg(a.Fa + e), oa = ldg(a.Oa + e);
    if (PACKED) {
        const float* r = a.rec + (e / n) * (4 * static_cast<int64_t>(n)) + j;
        za = za + ldg(r);
        ia = ia + ldg(r + n);
        fa = fa + ldg(r + 2 * static_cast<int64_t>(n));
        oa = oa + ldg(r + 3 * static_cast<int64_t>(n));
    }
    LstmCell c;
    c.za = za; c.ia = ia; c.fa = fa; c.oa = oa;
    lstm_cell_forward(c, act, c_prev, a.pi[j], a.pf[j], a.po[j], a.bz[j], a.bi[j], a.bf[j], a.bo[j]);
    za = c.za; ia = c.ia; fa = c.fa; oa = c.oa;
    const float zb = c.zb, ib = c.ib, fb = c.fb, ca = c.ca, ob = c.ob, cb = c.cb;
    stg(a.Za + e, za); stg(a.Zb + e, zb); stg(a.Ia + e, ia); stg(a.Ib + e, ib); stg(a.Fa + e, fa); stg(a.Fb + e, fb);
    stg(a.Ca + e, ca); stg(a.Oa + e, oa); stg(a.Ob + e, ob); stg(a.Cb + e, cb);
    a.y[e] = c.y;
}

struct LstmBwdArgs {
    const float *dy, *Zb, *Ib, *Fb, *Ob, *Cb, *Ca_prev, *Fb_next, *dIa_next, *dFa_next, *dCa_next;
    float *dZa, *dZb, *dIa, *dIb, *dFa, *dFb, *dOa, *dOb, *dCa, *dCb;
    const float *pi, *pf, *po;
    // PACKED only: dy holds the recurrent product packed[t+1] [Rz;Ri;Rf;Ro] on entry and
    // deltas[t] + that on return; packed_out (batch, 4n) receives [dZa|dIa|dFa|dOa] of this step
    const float* deltas;
    float* dy_out;
    float* packed_out;
};

struct LstmBwdCell { float dob, doa, dcb, dca, dfb, dfa, dib, dia, dzb, dza; };

// The backward step's arithmetic for element e (column j), given dy = deltas + recurrent deltas; shared by
// the step kernels so that all of them apply the same float32 operations in the same order.
__device__ __forceinline__ LstmBwdCell lstm_cell_backward(const LstmBwdArgs& a, int act, int64_t e, unsigned j, float dy) {
    LstmBwdCell c;
    float dca = ldg(a.dCa + e);
    { const float p = ldg(a.dIa_next + e) * a.pi[j]; dca = dca + p; }
    { const float p = ldg(a.dFa_next + e) * a.pf[j]; dca = dca + p; }
    const float ob = ldg(a.Ob + e), cb = ldg(a.Cb + e);
    c.dob = dy * cb;
    c.doa = SigmoidDerivOp{}.apply(ob, c.dob, 0.0f);
    { const float p = c.doa * a.po[j]; dca = dca + p; }
    float dcb = dy * ob;
    dcb = act_backward(act, cb, dcb);
    c.dcb = dcb;
    dca = dca + dcb;
    { const float p = ldg(a.dCa_next + e) * ldg(a.Fb_next + e); dca = dca + p; }
    c.dca = dca;
    c.dfb = dca * ldg(a.Ca_prev + e);
    c.dfa = SigmoidDerivOp{}.apply(ldg(a.Fb + e), c.dfb, 0.0f);
    const float zb = ldg(a.Zb + e), ib = ldg(a.Ib + e);
    c.dib = dca * zb;
    c.dia = SigmoidDerivOp{}.apply(ib, c.dib, 0.0f);
    c.dzb = dca * ib;
    c.dza = act_backward(act, zb, c.dzb);
    return c;
}

// The elementwise part of one LSTM backward time step (lstm_layer.py:180-205),
// after the recurrent deltas have been accumulated into dy:
//   mult_add_mv(dIa_next, pi, dCa); mult_add_mv(dFa_next, pf, dCa)
//   dOb = dy * Cb; dOa = sigmoid_deriv(Ob, dOb); mult_add_mv(dOa, po, dCa)
//   dCb = dy * Ob; dCb = act_deriv(Cb, dCb); dCa = dCa + dCb; mult_add_tt(dCa_next, Fb_next, dCa)
//   dFb = dCa * Ca_prev; dFa = sigmoid_deriv(Fb, dFb)
//   dIb = dCa * Zb;      dIa = sigmoid_deriv(Ib, dIb)
//   dZb = dCa * Ib;      dZa = act_deriv(Zb, dZb)
template <bool PACKED>
__global__ __launch_bounds__(kBlock) void lstm_bwd_step_kernel(LstmBwdArgs a, int act, int64_t total,
                                                               unsigned n) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const unsigned j = static_cast<unsigned>(e % n);
    float dy = ldg(a.dy + e);
    if (PACKED && a.deltas != nullptr) {     // without deltas, dy is complete already and only the packed copy is added
        dy = ldg(a.deltas + e) + dy;
        a.dy_out[e] = dy;
    }
    const LstmBwdCell c = lstm_cell_backward(a, act, e, j, dy);
    const float dob = c.dob, doa = c.doa, dcb = c.dcb, dca = c.dca, dfb = c.dfb, dfa = c.dfa, dib = c.dib, dia = c.dia,
                dzb = c.dzb, dza = c.dza;
    // the gate deltas feed the matrix products that follow and dCa the next step: those stay cached
    stg(a.dOb + e, dob); a.dOa[e] = doa; stg(a.dCb + e, dcb); a.dCa[e] = dca; stg(a.dFb + e, dfb); a.dFa[e] = dfa;
    stg(a.dIb + e, dib); a.dIa[e] = dia; stg(a.dZb + e, dzb); a.dZa[e] = dza;
    if (PACKED) {
        float* q = a.packed_out + (e / n) * (4 * static_cast<int64_t>(n)) + j;
        q[0] = dza;
        q[n] = dia;
        q[2 * static_cast<int64_t>(n)] = dfa;
        q[3 * static_cast<int64_t>(n)] = doa;
    }
}


// The backward step behind bship_dot_small_tn_f32: the recurrent deltas arrive as `parts` partial
// products (slabs of (batch, n), `part_stride` floats apart) that are added here in ascending order, and
// [dZa|dIa|dFa|dOa] leaves TRANSPOSED, as the (4n, 128) left operand of the next step's product
// (row g*n + j, column b; columns >= batch are never written). A workgroup owns an 8 x 32 tile of (batch, n),
// one element per lane; the four gate deltas turn through LDS and leave as 32-byte pieces of the operand's rows.
constexpr int kThinMaxParts = 8;

struct LstmBwdThinArgs {
    LstmBwdArgs s;               // s.dy = the partial products, s.packed_out = the transposed operand
    int parts;
    int64_t part_stride;
};

// PARTS: the number of slabs when it is 1, 2 or 4; 8 stands for "up to 8" (a slab beyond the last one reads the
// last one again and is not added).
template <int PARTS>
__global__ __launch_bounds__(256) void lstm_bwd_step_thin_kernel(LstmBwdThinArgs t, int act, int batch, unsigned n,
                                                                 unsigned col_tiles) {
    __shared__ float turn[4][8][33];
    const LstmBwdArgs& a = t.s;
    const int tid = static_cast<int>(threadIdx.x);
    const int b0 = static_cast<int>(blockIdx.x / col_tiles) * 8;
    const unsigned j0 = (blockIdx.x % col_tiles) * 32u;
    {
        const int tx = tid & 31, ty = tid >> 5;
        const int b = b0 + ty;
        const unsigned j = j0 + tx;
        if (b < batch && j < n) {
            const int64_t e = static_cast<int64_t>(b) * n + j;
            // all partial products are requested before the first is used
            float part[PARTS];
#pragma unroll
            for (int p = 0; p < PARTS; ++p)
                part[p] = ldg(a.dy + (PARTS < kThinMaxParts || p < t.parts ? p : t.parts - 1) * t.part_stride + e);
            float rec = part[0];
#pragma unroll
            for (int p = 1; p < PARTS; ++p) rec = (PARTS < kThinMaxParts || p < t.parts) ? rec + part[p] : rec;
            const float dy = ldg(a.deltas + e) + rec;
            a.dy_out[e] = dy;
            const LstmBwdCell c = lstm_cell_backward(a, act, e, j, dy);
            stg(a.dOb + e, c.dob); a.dOa[e] = c.doa; stg(a.dCb + e, c.dcb); a.dCa[e] = c.dca; stg(a.dFb + e, c.dfb);
            a.dFa[e] = c.dfa; stg(a.dIb + e, c.dib); a.dIa[e] = c.dia; stg(a.dZb + e, c.dzb); a.dZa[e] = c.dza;
            turn[0][ty][tx] = c.dza; turn[1][ty][tx] = c.dia; turn[2][ty][tx] = c.dfa; turn[3][ty][tx] = c.doa;
        }
    }
    __syncthreads();
    const int bb = tid & 7;
    const unsigned jj = static_cast<unsigned>(tid >> 3);
    if (b0 + bb < batch && j0 + jj < n) {
#pragma unroll
        for (int gate = 0; gate < 4; ++gate)
            a.packed_out[(static_cast<int64_t>(gate) * n + j0 + jj) * 128 + b0 + bb] = turn[gate][bb][jj];
    }
}

// =================== generic multi-operand streaming kernels ===================
// Bodies describe one element: apply(v, in, out) with v = the row-vector operands
// at this column, in = the matrix operands at this element, out = the results.
// A body provides the pointer tables vecs[kVecs], ins[kIn], outs[kOut]; an output
// may be the same array as an input (every lane loads all operands first).
constexpr int kFusedRows = 2;   // as kMvRows of the matrix-vector kernels

template <int W, bool AL, typename Body>
__global__ __launch_bounds__(kBlock) void rowvec_fused_kernel(Body b, int64_t M, int64_t NW,
                                                              unsigned col_tiles, bool through) {
    typedef typename VecT<W>::type T;
    constexpr int KV = Body::kVecs > 0 ? Body::kVecs : 1;
    constexpr int R = kFusedRows;
    const unsigned ct = blockIdx.x % col_tiles;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x / col_tiles) * R;
    const int64_t c = static_cast<int64_t>(ct) * kBlock + threadIdx.x;
    if (c >= NW) return;
    T v[KV];
#pragma unroll
    for (int k = 0; k < Body::kVecs; ++k) v[k] = vload<W, AL>(b.vecs[k] + c * W);
    T in[R][Body::kIn];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if (r0 + u < M) {
            const int64_t e = ((r0 + u) * NW + c) * W;
#pragma unroll
            for (int k = 0; k < Body::kIn; ++k) in[u][k] = vload<W, AL>(b.ins[k] + e);
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if (r0 + u < M) {
            const int64_t e = ((r0 + u) * NW + c) * W;
            T o[Body::kOut];
            if constexpr (W == 1) {
                float vs[KV], is[Body::kIn], os[Body::kOut];
#pragma unroll
                for (int k = 0; k < Body::kVecs; ++k) vs[k] = v[k];
#pragma unroll
                for (int k = 0; k < Body::kIn; ++k) is[k] = in[u][k];
                b.apply(vs, is, os);
#pragma unroll
                for (int k = 0; k < Body::kOut; ++k) o[k] = os[k];
            } else {
#pragma unroll
                for (int q = 0; q < W; ++q) {
                    float vs[KV], is[Body::kIn], os[Body::kOut];
#pragma unroll
                    for (int k = 0; k < Body::kVecs; ++k) vs[k] = v[k][q];
#pragma unroll
                    for (int k = 0; k < Body::kIn; ++k) is[k] = in[u][k][q];
                    b.apply(vs, is, os);
#pragma unroll
                    for (int k = 0; k < Body::kOut; ++k) o[k][q] = os[k];
                }
            }
#pragma unroll
            for (int k = 0; k < Body::kOut; ++k) vstore<W, AL>(b.outs[k] + e, o[k], through);
        }
    }
}

template <typename Body>
int launch_rowvec_fused(const char* name, const Body& b, int64_t M, int64_t N) {
    if (M == 0 || N == 0) return 0;
    const bool vec = (N % 4 == 0);
    const int64_t NW = vec ? N / 4 : N;
    const int64_t col_tiles = ceil_div(NW, kBlock);
    const int64_t blocks = col_tiles * ceil_div(M, kFusedRows);
    if (blocks > 0x7fffffff)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: matrix too large for one launch", name);
    bool al = true;
    for (int k = 0; k < Body::kVecs; ++k) al = al && aligned16(b.vecs[k]);
    for (int k = 0; k < Body::kIn; ++k) al = al && aligned16(b.ins[k]);
    for (int k = 0; k < Body::kOut; ++k) al = al && aligned16(b.outs[k]);
    const dim3 grid(static_cast<unsigned>(blocks)), blk(kBlock);
    const unsigned ctl = static_cast<unsigned>(col_tiles);
    hipStream_t s = ctx().stream;
    const bool through = store_through(static_cast<size_t>(M) * static_cast<size_t>(N));
    // (runs of adjacent tiles per XCD, which help the flat kernels below, cost these 2-4 %: measured on
    // the batch normalisation passes at 2048 x 4096 and 8192 x 8192)
    if (vec && al) hipLaunchKernelGGL((rowvec_fused_kernel<4, true, Body>), grid, blk, 0, s, b, M, NW, ctl, through);
    else if (vec)  hipLaunchKernelGGL((rowvec_fused_kernel<4, false, Body>), grid, blk, 0, s, b, M, NW, ctl, through);
    else           hipLaunchKernelGGL((rowvec_fused_kernel<1, false, Body>), grid, blk, 0, s, b, M, NW, ctl, through);
    return check_launch(name);
}

// Flat arrays: one workgroup per tile of 1024 floats, one 128-bit vector per lane
// and operand; the array's last, partial vector is handled element by element.
template <bool AL, typename Body>
__global__ __launch_bounds__(kBlock) void flat_fused_kernel(Body b, size_t n, unsigned run, bool through) {
    const size_t i = (static_cast<size_t>(xcd_run_tile(run)) * kBlock + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {
        f4 in[Body::kIn], o[Body::kOut];
#pragma unroll
        for (int k = 0; k < Body::kIn; ++k) in[k] = vload<4, AL>(b.ins[k] + i);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float is[Body::kIn], os[Body::kOut];
#pragma unroll
            for (int k = 0; k < Body::kIn; ++k) is[k] = in[k][q];
            b.apply(nullptr, is, os);
#pragma unroll
            for (int k = 0; k < Body::kOut; ++k) o[k][q] = os[k];
        }
#pragma unroll
        for (int k = 0; k < Body::kOut; ++k) vstore<4, AL>(b.outs[k] + i, o[k], through);
    } else {
        for (size_t j = i; j < n; ++j) {
            float is[Body::kIn], os[Body::kOut];
#pragma unroll
            for (int k = 0; k < Body::kIn; ++k) is[k] = b.ins[k][j];
            b.apply(nullptr, is, os);
#pragma unroll
            for (int k = 0; k < Body::kOut; ++k) b.outs[k][j] = os[k];
        }
    }
}

template <typename Body>
int launch_flat_fused(const char* name, const Body& b, size_t n) {
    if (n == 0) return 0;
    const size_t tiles = (n + static_cast<size_t>(kBlock) * 4 - 1) / (static_cast<size_t>(kBlock) * 4);
    if (tiles > 0x7fffffffu)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: %zu elements exceed one launch", name, n);
    bool al = true;
    for (int k = 0; k < Body::kIn; ++k) al = al && aligned16(b.ins[k]);
    for (int k = 0; k < Body::kOut; ++k) al = al && aligned16(b.outs[k]);
    const dim3 grid(static_cast<unsigned>(tiles)), blk(kBlock);
    // three or more streams: an XCD takes runs of adjacent tiles, as in the elementwise kernels
    const unsigned run = Body::kIn + Body::kOut >= 3 ? static_cast<unsigned>(ctx().ew_run_bytes / (kBlock * 4 * sizeof(float))) : 0;
    if (al) hipLaunchKernelGGL((flat_fused_kernel<true, Body>), grid, blk, 0, ctx().stream, b, n, run, store_through(n));
    else    hipLaunchKernelGGL((flat_fused_kernel<false, Body>), grid, blk, 0, ctx().stream, b, n, run, store_through(n));
    return check_launch(name);
}

// ---- Highway (highway_layer.py:40-71) ----
// forward:  tmp = H - x; tmp = T * tmp; y = tmp + x
struct HighwayFwdBody {
    static constexpr int kVecs = 0, kIn = 3, kOut = 1;
    const float* ins[3];   // H, T, x
    float* outs[1];        // y
    __device__ void apply(const float*, const float* in, float* o) const {
        float tmp = in[0] - in[2];
        tmp = in[1] * tmp;
        o[0] = tmp + in[2];
    }
};
// backward: tmp = 1 - T; dx += tmp * dy; dH += T * dy; tmp = H - x; dT += tmp * dy
struct HighwayBwdBody {
    static constexpr int kVecs = 0, kIn = 7, kOut = 3;
    const float* ins[7];   // H, T, x, dy, dx, dH, dT
    float* outs[3];        // dx, dH, dT
    __device__ void apply(const float*, const float* in, float* o) const {
        const float dy = in[3];
        float tmp = 1.0f - in[1];
        o[0] = MultAddOp{}.apply(tmp, dy, in[4]);
        o[1] = MultAddOp{}.apply(in[1], dy, in[5]);
        tmp = in[0] - in[2];
        o[2] = MultAddOp{}.apply(tmp, dy, in[6]);
    }
};

// ---- momentum update (steppers.py:104-114) ----
// velocity = momentum * velocity; velocity += (-learning_rate) * gradients; parameters = velocity + parameters
struct MomentumBody {
    static constexpr int kVecs = 0, kIn = 3, kOut = 2;
    const float* ins[3];   // gradients, velocity, parameters
    float* outs[2];        // velocity, parameters
    float momentum, neg_learning_rate;
    __device__ void apply(const float*, const float* in, float* o) const {
        float v = MultStOp{momentum}.apply(in[1], 0.0f, 0.0f);
        v = MultAddStOp{neg_learning_rate}.apply(in[0], v, 0.0f);
        o[0] = v;
        o[1] = AddOp{}.apply(v, in[2], 0.0f);
    }
};

// ---- softmax cross entropy (softmax_ce_layer.py:65-114) ----
// forward, behind softmax_m: loss[i] = -1 * log(clip(probs[i, int(targets[i])], 1e-6, 1))
// (index_m_by_v, clip_t, log_t, mult_st; the layer's fill(loss, 0) is overwritten by them)
__global__ __launch_bounds__(kBlock) void softmax_ce_loss_kernel(const float* __restrict__ probs,
                                                                 const float* __restrict__ targets,
                                                                 float* __restrict__ loss, int64_t M, int64_t K) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (row >= M) return;
    const int64_t j = label_column(targets[row], K);
    float p = j >= 0 ? probs[row * K + j] : 0.0f;
    p = ClipOp{1e-6f, 1.0f}.apply(p, 0.0f, 0.0f);
    p = LogOp{}.apply(p, 0.0f, 0.0f);
    loss[row] = MultStOp{-1.0f}.apply(p, 0.0f, 0.0f);
}
// backward: t = onehot(targets); t = -1 * t; t = t + probs; t = t * dloss[row]; t_bin = t;
// dinputs = t + dinputs   (binarize_v, mult_st, add_tt, mult_mv, add_tt)
__global__ __launch_bounds__(kBlock) void softmax_ce_bwd_kernel(const float* __restrict__ probs,
                                                                const float* __restrict__ targets,
                                                                const float* __restrict__ dloss,
                                                                float* __restrict__ t_bin, float* dinputs,
                                                                int64_t total, int64_t K) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= total) return;
    const int64_t row = i / K;
    const int64_t j = i - row * K;
    float t = (j == label_column(targets[row], K)) ? 1.0f : 0.0f;
    t = MultStOp{-1.0f}.apply(t, 0.0f, 0.0f);
    t = AddOp{}.apply(t, probs[i], 0.0f);
    t = MulOp{}.apply(t, dloss[row], 0.0f);
    t_bin[i] = t;
    dinputs[i] = AddOp{}.apply(t, dinputs[i], 0.0f);
}

// ---- bias + activation of a fully connected layer (fully_connected_layer.py:62-64) ----
template <typename Act>
struct BiasActBody {
    static constexpr int kVecs = 1, kIn = 1, kOut = 1;
    const float* vecs[1];  // bias
    const float* ins[1];   // the matrix product
    float* outs[1];
    __device__ void apply(const float* v, const float* in, float* o) const {
        const float z = in[0] + v[0];
        o[0] = Act{}.apply(z, 0.0f, 0.0f);
    }
};
struct LinearOp { __device__ float apply(float x, float, float) const { return x; } };

// ---- batch normalisation (batch_normalization_layer.py:54-152) ----
// source of the variance reduction: centered = x + mu_b (stored), value = centered^2
struct CenterSquareSrc {
    const float* x;
    const float* mu;
    float* centered;
    bool through;           // store centered write-through (store_through of the matrix size)
    bool aligned() const { return aligned16(x) && aligned16(mu) && aligned16(centered); }
    template <int W, bool AL> __device__ typename VecT<W>::type prep(int64_t col) const {
        return vload<W, AL>(mu + col);
    }
    template <int W, bool AL>
    __device__ typename VecT<W>::type load(int64_t off, typename VecT<W>::type m) const {
        const typename VecT<W>::type c = vload<W, AL>(x + off) + m;
        vstore<W, AL>(centered + off, c, through);
        return c * c;
    }
};
// source of the dgamma reduction: out_deltas * x_hat
struct ProductSrc {
    const float* a;
    const float* b;
    bool aligned() const { return aligned16(a) && aligned16(b); }
    template <int W, bool AL> __device__ typename VecT<W>::type prep(int64_t) const {
        return vzero<typename VecT<W>::type>();
    }
    template <int W, bool AL>
    __device__ typename VecT<W>::type load(int64_t off, typename VecT<W>::type) const {
        return vload<W, AL>(a + off) * vload<W, AL>(b + off);
    }
};

// mu_b = (-1/m) * colsum; mu = decay * mu; mu += (1 - decay) * mu_b
__global__ __launch_bounds__(kBlock) void bn_mean_update_kernel(float* mu_b, float* mu, float neg_inv_m,
                                                                float decay, float one_minus_decay,
                                                                int64_t n) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (j >= n) return;
    const float b = MultStOp{neg_inv_m}.apply(mu_b[j], 0.0f, 0.0f);
    mu_b[j] = b;
    const float r = MultStOp{decay}.apply(mu[j], 0.0f, 0.0f);
    mu[j] = MultAddStOp{one_minus_decay}.apply(b, r, 0.0f);
}

// sigma2 = (1/m) * colsum; sigma2 += eps; sigma_b = sqrt(sigma2);
// sigma = decay * sigma; sigma += (1 - decay) * sigma_b
__global__ __launch_bounds__(kBlock) void bn_sigma_update_kernel(float* sigma_b, float* sigma, float inv_m,
                                                                 float eps, float decay,
                                                                 float one_minus_decay, int64_t n) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (j >= n) return;
    float s2 = MultStOp{inv_m}.apply(sigma_b[j], 0.0f, 0.0f);
    s2 = AddStOp{eps}.apply(s2, 0.0f, 0.0f);
    const float sb = SqrtOp{}.apply(s2, 0.0f, 0.0f);
    sigma_b[j] = sb;
    const float r = MultStOp{decay}.apply(sigma[j], 0.0f, 0.0f);
    sigma[j] = MultAddStOp{one_minus_decay}.apply(sb, r, 0.0f);
}

// dgamma += s1; s1 *= 1/m; dbeta += s2; s2 *= 1/m; coeff = gamma / sigma_b
__global__ __launch_bounds__(kBlock) void bn_bwd_vectors_kernel(float* s1, float* s2, float* coeff,
                                                                float* dgamma, float* dbeta,
                                                                const float* gamma, const float* sigma_b,
                                                                float inv_m, int64_t n) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (j >= n) return;
    const float a = s1[j], b = s2[j];
    dgamma[j] = a + dgamma[j];
    s1[j] = MultStOp{inv_m}.apply(a, 0.0f, 0.0f);
    dbeta[j] = b + dbeta[j];
    s2[j] = MultStOp{inv_m}.apply(b, 0.0f, 0.0f);
    coeff[j] = gamma[j] / sigma_b[j];
}

// x_hat = centered / sigma; out = x_hat * gamma; out += beta
struct BnNormBody {
    static constexpr int kVecs = 3, kIn = 1, kOut = 2;
    const float* vecs[3];  // sigma, gamma, beta
    const float* ins[1];   // centered
    float* outs[2];        // x_hat, out
    __device__ void apply(const float* v, const float* in, float* o) const {
        const float xh = in[0] / v[0];
        const float t = xh * v[1];
        o[0] = xh;
        o[1] = t + v[2];
    }
};
// the same with the centering in front (inference: running mean and deviation)
struct BnInferBody {
    static constexpr int kVecs = 4, kIn = 1, kOut = 3;
    const float* vecs[4];  // mu (negative running mean), sigma, gamma, beta
    const float* ins[1];   // inputs
    float* outs[3];        // centered, x_hat, out
    __device__ void apply(const float* v, const float* in, float* o) const {
        const float c = in[0] + v[0];
        const float xh = c / v[1];
        const float t = xh * v[2];
        o[0] = c;
        o[1] = xh;
        o[2] = t + v[3];
    }
};
// term1 = x_hat * s1; term2 = dy - term1; term3 = term2 - s2; term4 = term3 * coeff;
// in_deltas = term4 + in_deltas
struct BnBwdBody {
    static constexpr int kVecs = 3, kIn = 3, kOut = 1;
    const float* vecs[3];  // s1 = colsum(dy * x_hat) / m, s2 = colsum(dy) / m, coeff = gamma / sigma_b
    const float* ins[3];   // out_deltas, x_hat, in_deltas
    float* outs[1];        // in_deltas
    __device__ void apply(const float* v, const float* in, float* o) const {
        const float t1 = in[1] * v[0];
        const float t2 = in[0] - t1;
        const float t3 = t2 - v[1];
        const float t4 = t3 * v[2];
        o[0] = t4 + in[2];
    }
};
}  // namespace bship

namespace bship {
namespace {

int check_pointers(const char* fn, const void* const* ptrs, int count) {
    for (int i = 0; i < count; ++i) {
        if (ptrs[i] == nullptr) return set_error(BSHIP_ERR_NULL_POINTER, "%s: an argument is NULL", fn);
        if (reinterpret_cast<uintptr_t>(ptrs[i]) & 3u)
            return set_error(BSHIP_ERR_BAD_POINTER, "%s: an argument is not 4-byte aligned", fn);
    }
    return 0;
}

int check_step_args(const char* fn, int act, int64_t batch, int64_t n, const void* const* ptrs,
                    int count) {
    if (!ctx().inited)
        return set_error(BSHIP_ERR_NOT_INITIALIZED, "%s: bship_init() has not been called", fn);
    BSHIP_FLUSH_PENDING();
    if (batch < 0 || n < 0 || n > 0x3fffffff)
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: bad dimensions batch=%lld n=%lld", fn,
                         (long long)batch, (long long)n);
    if (act < kActSigmoid || act > kActEl)
        return set_error(BSHIP_ERR_BAD_OP, "%s: unknown activation %d", fn, act);
    if (batch * n == 0) return 0;
    for (int i = 0; i < count; ++i) {
        if (ptrs[i] == nullptr) return set_error(BSHIP_ERR_NULL_POINTER, "%s: an argument is NULL", fn);
        if (reinterpret_cast<uintptr_t>(ptrs[i]) & 3u)
            return set_error(BSHIP_ERR_BAD_POINTER, "%s: an argument is not 4-byte aligned", fn);
    }
    return 0;
}

int lstm_fwd_launch(const char* fn, bool packed, int act, int64_t batch, int64_t n,
                    const LstmFwdArgs& a) {
    const void* ptrs[] = {a.Za, a.Zb, a.Ia, a.Ib, a.Fa, a.Fb, a.Oa, a.Ob, a.Ca, a.Cb, a.y, a.Ca_prev,
                          a.pi, a.pf, a.po, a.bz, a.bi, a.bf, a.bo, a.rec};
    int st = check_step_args(fn, act, batch, n, ptrs, packed ? 20 : 19);
    const int64_t total = batch * n;
    if (st != 0 || total == 0) return st;
    const dim3 grid(static_cast<unsigned>(ceil_div(total, kBlock)));
    if (packed)
        hipLaunchKernelGGL(lstm_fwd_step_kernel<true>, grid, dim3(kBlock), 0, ctx().stream, a, act,
                           total, static_cast<unsigned>(n));
    else
        hipLaunchKernelGGL(lstm_fwd_step_kernel<false>, grid, dim3(kBlock), 0, ctx().stream, a, act,
                           total, static_cast<unsigned>(n));
    return check_launch("lstm_forward_step");
}

int lstm_bwd_launch(const char* fn, bool packed, int act, int64_t batch, int64_t n,
                    const LstmBwdArgs& a) {
    const void* ptrs[] = {a.dy, a.Zb, a.Ib, a.Fb, a.Ob, a.Cb, a.Ca_prev, a.Fb_next, a.dIa_next,
                          a.dFa_next, a.dCa_next, a.dZa, a.dZb, a.dIa, a.dIb, a.dFa, a.dFb, a.dOa,
                          a.dOb, a.dCa, a.dCb, a.pi, a.pf, a.po, a.deltas ? a.deltas : a.dy, a.packed_out};
    int st = check_step_args(fn, act, batch, n, ptrs, packed ? 26 : 24);
    const int64_t total = batch * n;
    if (st != 0 || total == 0) return st;
    const dim3 grid(static_cast<unsigned>(ceil_div(total, kBlock)));
    if (packed)
        hipLaunchKernelGGL(lstm_bwd_step_kernel<true>, grid, dim3(kBlock), 0, ctx().stream, a, act,
                           total, static_cast<unsigned>(n));
    else
        hipLaunchKernelGGL(lstm_bwd_step_kernel<false>, grid, dim3(kBlock), 0, ctx().stream, a, act,
                           total, static_cast<unsigned>(n));
    return check_launch("lstm_backward_step");
}

}  // namespace

// batch_normalization_layer.py:68-105 for a training pass; the scalars are the ones the layer's calls carry
// (mult_st(-1/m), mult_st(decay), mult_add_st(1-decay) for the mean; mult_st(1/m), add_st(eps), mult_st(decay),
// mult_add_st(1-decay) for the deviation).
int batchnorm_fwd_train_launch(const float* inputs, const float* gamma, const float* beta, float* mu, float* sigma,
                               float* sigma_b, float* centered, float* x_hat, float* out, int64_t M, int64_t N,
                               float neg_inv_m, float decay_mu, float rest_mu, float inv_m, float eps,
                               float decay_sigma, float rest_sigma) {
    if (N == 0) return 0;
    if (M < 1) return set_error(BSHIP_ERR_BAD_DIMENSION, "batchnorm_forward: no rows");
    const dim3 vgrid(static_cast<unsigned>(ceil_div(N, kBlock))), blk(kBlock);
    hipStream_t s = ctx().stream;
    // negative batch mean into sigma_b (the layer uses that buffer as scratch), running mean
    int st = M == 1 ? bship_d2d(sigma_b, inputs, static_cast<size_t>(N) * 4)
                    : launch_colsum(PlainSrc{inputs}, sigma_b, M, N);
    if (st != 0) return st;
    hipLaunchKernelGGL(bn_mean_update_kernel, vgrid, blk, 0, s, sigma_b, mu, neg_inv_m, decay_mu, rest_mu, N);
    if ((st = check_launch("batchnorm mean")) != 0) return st;
    // centered = inputs + mu_b while summing centered^2 down the columns
    st = launch_colsum(CenterSquareSrc{inputs, sigma_b, centered,
                                       store_through(static_cast<size_t>(M) * static_cast<size_t>(N))}, sigma_b, M, N);
    if (st != 0) return st;
    hipLaunchKernelGGL(bn_sigma_update_kernel, vgrid, blk, 0, s, sigma_b, sigma, inv_m, eps, decay_sigma, rest_sigma, N);
    if ((st = check_launch("batchnorm deviation")) != 0) return st;
    BnNormBody b{{sigma_b, gamma, beta}, {centered}, {x_hat, out}};
    return launch_rowvec_fused("batchnorm_forward", b, M, N);
}

}  // namespace bship

using namespace bship;

extern "C" {

int bship_lstm_fwd_step_f32(int act, int64_t batch, int64_t n, float* Za, float* Zb, float* Ia,
                            float* Ib, float* Fa, float* Fb, float* Oa, float* Ob, float* Ca,
                            float* Cb, const float* Ca_prev, float* y, const float* pi,
                            const float* pf, const float* po, const float* bz, const float* bi,
                            const float* bf, const float* bo) {
    LstmFwdArgs a{Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y, Ca_prev, pi, pf, po, bz, bi, bf, bo, nullptr};
    return lstm_fwd_launch(__func__, false, act, batch, n, a);
}

int bship_lstm_fwd_step_packed_f32(int act, int64_t batch, int64_t n, const float* rec, float* Za,
                                   float* Zb, float* Ia, float* Ib, float* Fa, float* Fb, float* Oa,
                                   float* Ob, float* Ca, float* Cb, const float* Ca_prev, float* y,
                                   const float* pi, const float* pf, const float* po,
                                   const float* bz, const float* bi, const float* bf,
                                   const float* bo) {
    LstmFwdArgs a{Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y, Ca_prev, pi, pf, po, bz, bi, bf, bo, rec};
    return lstm_fwd_launch(__func__, true, act, batch, n, a);
}

int bship_lstm_bwd_step_f32(int act, int64_t batch, int64_t n, const float* dy, const float* Zb,
                            const float* Ib, const float* Fb, const float* Ob, const float* Cb,
                            const float* Ca_prev, const float* Fb_next, const float* dIa_next,
                            const float* dFa_next, const float* dCa_next, float* dZa, float* dZb,
                            float* dIa, float* dIb, float* dFa, float* dFb, float* dOa, float* dOb,
                            float* dCa, float* dCb, const float* pi, const float* pf,
                            const float* po) {
    LstmBwdArgs a{dy, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                  dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po,
                  nullptr, nullptr, nullptr};
    return lstm_bwd_launch(__func__, false, act, batch, n, a);
}

int bship_lstm_bwd_step_packed_f32(int act, int64_t batch, int64_t n, const float* deltas, float* dy,
                                   float* packed_out, const float* Zb, const float* Ib,
                                   const float* Fb, const float* Ob, const float* Cb,
                                   const float* Ca_prev, const float* Fb_next, const float* dIa_next,
                                   const float* dFa_next, const float* dCa_next, float* dZa,
                                   float* dZb, float* dIa, float* dIb, float* dFa, float* dFb,
                                   float* dOa, float* dOb, float* dCa, float* dCb, const float* pi,
                                   const float* pf, const float* po) {
    LstmBwdArgs a{dy, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                  dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po,
                  deltas, dy, packed_out};
    return lstm_bwd_launch(__func__, true, act, batch, n, a);
}

int bship_lstm_bwd_step_thin_f32(int act, int64_t batch, int64_t n, const float* deltas, const float* dy_parts,
                                 int parts, int64_t part_stride, float* dy, float* packed_t_out, const float* Zb,
                                 const float* Ib, const float* Fb, const float* Ob, const float* Cb,
                                 const float* Ca_prev, const float* Fb_next, const float* dIa_next,
                                 const float* dFa_next, const float* dCa_next, float* dZa, float* dZb, float* dIa,
                                 float* dIb, float* dFa, float* dFb, float* dOa, float* dOb, float* dCa, float* dCb,
                                 const float* pi, const float* pf, const float* po) {
    LstmBwdThinArgs t{{dy_parts, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                       dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po, deltas, dy, packed_t_out},
                      parts, part_stride};
    const void* ptrs[] = {dy_parts, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next, dZa, dZb, dIa,
                          dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po, deltas, dy, packed_t_out};
    int st = check_step_args(__func__, act, batch, n, ptrs, 27);
    if (st != 0 || batch * n == 0) return st;
    if (batch > 128 || parts < 1 || parts > kThinMaxParts || (parts > 1 && part_stride < batch * n))
        return set_error(BSHIP_ERR_BAD_DIMENSION, "%s: batch %lld (at most 128), parts %d (1..8), part_stride %lld",
                         __func__, (long long)batch, parts, (long long)part_stride);
    const int64_t row_tiles = ceil_div(batch, 8), col_tiles = ceil_div(n, 32);
    const dim3 grid(static_cast<unsigned>(row_tiles * col_tiles));
#define BSHIP_THIN_STEP(P_)                                                                                        \
    hipLaunchKernelGGL(lstm_bwd_step_thin_kernel<P_>, grid, dim3(256), 0, ctx().stream, t, act, static_cast<int>(batch), \
                       static_cast<unsigned>(n), static_cast<unsigned>(col_tiles))
    switch (parts) {
        case 1: BSHIP_THIN_STEP(1); break;
        case 2: BSHIP_THIN_STEP(2); break;
        case 4: BSHIP_THIN_STEP(4); break;
        default: BSHIP_THIN_STEP(8); break;
    }
#undef BSHIP_THIN_STEP
    return check_launch("lstm_backward_step_thin");
}

int bship_highway_fwd_f32(const float* H, const float* T, const float* x, float* y, size_t n) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    const void* ptrs[] = {H, T, x, y};
    int st = check_pointers(__func__, ptrs, 4);
    if (st != 0) return st;
    HighwayFwdBody b{{H, T, x}, {y}};
    return launch_flat_fused("highway_forward", b, n);
}

int bship_highway_bwd_f32(const float* H, const float* T, const float* x, const float* dy, float* dx,
                          float* dH, float* dT, size_t n) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    const void* ptrs[] = {H, T, x, dy, dx, dH, dT};
    int st = check_pointers(__func__, ptrs, 7);
    if (st != 0) return st;
    HighwayBwdBody b{{H, T, x, dy, dx, dH, dT}, {dx, dH, dT}};
    return launch_flat_fused("highway_backward", b, n);
}

int bship_momentum_update_f32(float momentum, float neg_learning_rate, const float* gradients, float* velocity,
                              float* parameters, size_t n) {
    BSHIP_REQUIRE_INIT();
    if (n == 0) return 0;
    const void* ptrs[] = {gradients, velocity, parameters};
    int st = check_pointers(__func__, ptrs, 3);
    if (st != 0) return st;
    MomentumBody b{{gradients, velocity, parameters}, {velocity, parameters}, momentum, neg_learning_rate};
    return launch_flat_fused("momentum_update", b, n);
}

int bship_softmax_ce_fwd_f32(const float* inputs, const float* targets, float* probs, float* loss, int64_t M,
                             int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    if (M == 0) return 0;
    const void* ptrs[] = {inputs, targets, probs, loss};
    int st = check_pointers(__func__, ptrs, 4);
    if (st != 0) return st;
    BSHIP_REQUIRE_DIM(M <= 0x7fffffff);
    st = bship_softmax_rows_pitched_f32(inputs, K, probs, K, M, K);     // not through the fusing window
    if (st != 0) return st;
    hipLaunchKernelGGL(softmax_ce_loss_kernel, dim3(static_cast<unsigned>(ceil_div(M, kBlock))), dim3(kBlock), 0,
                       ctx().stream, probs, targets, loss, M, K);
    return check_launch("softmax_ce_forward");
}

int bship_softmax_ce_bwd_f32(const float* probs, const float* targets, const float* dloss, float* t_bin,
                             float* dinputs, int64_t M, int64_t K) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && K >= 0);
    if (M == 0 || K == 0) return 0;
    const void* ptrs[] = {probs, targets, dloss, t_bin, dinputs};
    int st = check_pointers(__func__, ptrs, 5);
    if (st != 0) return st;
    const int64_t total = M * K;
    BSHIP_REQUIRE_DIM(ceil_div(total, kBlock) <= 0x7fffffff);
    hipLaunchKernelGGL(softmax_ce_bwd_kernel, dim3(static_cast<unsigned>(ceil_div(total, kBlock))), dim3(kBlock), 0,
                       ctx().stream, probs, targets, dloss, t_bin, dinputs, total, K);
    return check_launch("softmax_ce_backward");
}

int bship_bias_act_f32(int act, const float* in, const float* bias, float* out, int64_t M, int64_t N) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    if (act < kActSigmoid || act > kActEl)
        return set_error(BSHIP_ERR_BAD_OP, "%s: unknown activation %d", __func__, act);
    if (M == 0 || N == 0) return 0;
    const void* ptrs[] = {in, bias, out};
    int st = check_pointers(__func__, ptrs, 3);
    if (st != 0) return st;
    switch (act) {
        case kActSigmoid: return launch_rowvec_fused("bias_act", BiasActBody<SigmoidOp>{{bias}, {in}, {out}}, M, N);
        case kActTanh:    return launch_rowvec_fused("bias_act", BiasActBody<TanhOp>{{bias}, {in}, {out}}, M, N);
        case kActRel:     return launch_rowvec_fused("bias_act", BiasActBody<RelOp>{{bias}, {in}, {out}}, M, N);
        case kActEl:      return launch_rowvec_fused("bias_act", BiasActBody<ElOp>{{bias}, {in}, {out}}, M, N);
        default:          return launch_rowvec_fused("bias_act", BiasActBody<LinearOp>{{bias}, {in}, {out}}, M, N);
    }
}

int bship_batchnorm_fwd_f32(int training, const float* inputs, const float* gamma, const float* beta,
                            float* mu, float* sigma, double decay, double epsilon, float* sigma_b,
                            float* centered, float* x_hat, float* out, int64_t M, int64_t N) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 0 && N >= 0);
    if (N == 0) return 0;
    const void* ptrs[] = {inputs, gamma, beta, mu, sigma, sigma_b, centered, x_hat, out};
    int st = check_pointers(__func__, ptrs, 9);
    if (st != 0) return st;
    if (!training) {
        BnInferBody b{{mu, sigma, gamma, beta}, {inputs}, {centered, x_hat, out}};
        return launch_rowvec_fused("batchnorm_forward", b, M, N);
    }
    BSHIP_REQUIRE_DIM(M >= 1);
    // Python evaluates -1.0/m, 1.0/m and 1.0-decay in double; the handler then rounds to float32
    const float neg_inv_m = static_cast<float>(-1.0 / static_cast<double>(M));
    const float inv_m = static_cast<float>(1.0 / static_cast<double>(M));
    const float dec = static_cast<float>(decay);
    const float omd = static_cast<float>(1.0 - decay);
    const float eps = static_cast<float>(epsilon);
    return batchnorm_fwd_train_launch(inputs, gamma, beta, mu, sigma, sigma_b, centered, x_hat, out, M, N,
                                      neg_inv_m, dec, omd, inv_m, eps, dec, omd);
}

int bship_batchnorm_bwd_f32(const float* out_deltas, const float* x_hat, const float* gamma,
                            const float* sigma_b, float* dgamma, float* dbeta, float* in_deltas,
                            int64_t M, int64_t N) {
    BSHIP_REQUIRE_INIT();
    BSHIP_REQUIRE_DIM(M >= 1 && N >= 0);
    if (N == 0) return 0;
    const void* ptrs[] = {out_deltas, x_hat, gamma, sigma_b, dgamma, dbeta, in_deltas};
    int st = check_pointers(__func__, ptrs, 7);
    if (st != 0) return st;
    void* raw = nullptr;
    const size_t vec_bytes = (static_cast<size_t>(N) * 4 + 255) & ~static_cast<size_t>(255);
    if ((st = pool_alloc_raw(3 * vec_bytes, &raw)) != 0) return st;
    float* s1 = static_cast<float*>(raw);
    float* s2 = reinterpret_cast<float*>(static_cast<char*>(raw) + vec_bytes);
    float* coeff = reinterpret_cast<float*>(static_cast<char*>(raw) + 2 * vec_bytes);
    const float inv_m = static_cast<float>(1.0 / static_cast<double>(M));
    st = launch_colsum(ProductSrc{out_deltas, x_hat}, s1, M, N);
    if (st == 0)
        st = M == 1 ? bship_d2d(s2, out_deltas, static_cast<size_t>(N) * 4)
                    : launch_colsum(PlainSrc{out_deltas}, s2, M, N);
    if (st == 0) {
        hipLaunchKernelGGL(bn_bwd_vectors_kernel, dim3(static_cast<unsigned>(ceil_div(N, kBlock))),
                           dim3(kBlock), 0, ctx().stream, s1, s2, coeff, dgamma, dbeta, gamma, sigma_b,
                           inv_m, N);
        st = check_launch("batchnorm gradients");
    }
    if (st == 0) {
        BnBwdBody b{{s1, s2, coeff}, {out_deltas, x_hat, in_deltas}, {in_deltas}};
        st = launch_rowvec_fused("batchnorm_backward", b, M, N);
    }
    pool_free_raw(raw);   // a later owner of the block runs after these launches
    return st;
}

}  // extern "C"
