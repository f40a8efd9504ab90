// Fused layer-level kernels: optional entry points that do in one launch what a
// brainstorm layer does with a dozen handler calls per time step. They are an
// extension, not part of the reference's handler interface; the primitive
// operations remain the default. Each kernel chains the very same per-element
// functors (functors.h) in the order the layer issues the primitive calls, so
// its results are bit-identical to the unfused sequence.
#pragma clang fp contract(off)

#include "common.h"
#include "functors.h"

namespace bship {

enum { kActSigmoid = 0, kActTanh = 1, kActRel = 2, kActLinear = 3, kActEl = 4 };

// act_func[...] (base_handler.py:57-63); 'linear' is copy_to
__device__ __forceinline__ float act_forward(int act, float x) {
    switch (act) {
        case kActSigmoid: return SigmoidOp{}.apply(x, 0.0f, 0.0f);
        case kActTanh:    return TanhOp{}.apply(x, 0.0f, 0.0f);
        case kActRel:     return RelOp{}.apply(x, 0.0f, 0.0f);
        case kActEl:      return ElOp{}.apply(x, 0.0f, 0.0f);
        default:          return x;
    }
}

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
template <bool PACKED>
__global__ __launch_bounds__(kBlock) void lstm_fwd_step_kernel(LstmFwdArgs a, int act, int64_t total,
                                                               unsigned n) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const unsigned j = static_cast<unsigned>(e % n);       // column: index into the (1,n) parameters
    const float c_prev = a.Ca_prev[e];
    float za = a.Za[e], ia = a.Ia[e], fa = a.Fa[e], oa = a.Oa[e];
    if (PACKED) {
        const float* r = a.rec + (e / n) * (4 * static_cast<int64_t>(n)) + j;
        za = za + r[0];
        ia = ia + r[n];
        fa = fa + r[2 * static_cast<int64_t>(n)];
        oa = oa + r[3 * static_cast<int64_t>(n)];
    }
    za = za + a.bz[j];
    const float zb = act_forward(act, za);
    { const float p = c_prev * a.pi[j]; ia = ia + p; }
    ia = ia + a.bi[j];
    const float ib = SigmoidOp{}.apply(ia, 0.0f, 0.0f);
    { const float p = c_prev * a.pf[j]; fa = fa + p; }
    fa = fa + a.bf[j];
    const float fb = SigmoidOp{}.apply(fa, 0.0f, 0.0f);
    float ca = ib * zb;
    { const float p = fb * c_prev; ca = ca + p; }
    { const float p = ca * a.po[j]; oa = oa + p; }
    oa = oa + a.bo[j];
    const float ob = SigmoidOp{}.apply(oa, 0.0f, 0.0f);
    const float cb = act_forward(act, ca);
    a.Za[e] = za; a.Zb[e] = zb; a.Ia[e] = ia; a.Ib[e] = ib; a.Fa[e] = fa; a.Fb[e] = fb;
    a.Ca[e] = ca; a.Oa[e] = oa; a.Ob[e] = ob; a.Cb[e] = cb;
    a.y[e] = ob * cb;
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
    float dy = a.dy[e];
    if (PACKED) {
        dy = a.deltas[e] + dy;
        a.dy_out[e] = dy;
    }
    float dca = a.dCa[e];
    { const float p = a.dIa_next[e] * a.pi[j]; dca = dca + p; }
    { const float p = a.dFa_next[e] * a.pf[j]; dca = dca + p; }
    const float ob = a.Ob[e], cb = a.Cb[e];
    const float dob = dy * cb;
    const float doa = SigmoidDerivOp{}.apply(ob, dob, 0.0f);
    { const float p = doa * a.po[j]; dca = dca + p; }
    float dcb = dy * ob;
    dcb = act_backward(act, cb, dcb);
    dca = dca + dcb;
    { const float p = a.dCa_next[e] * a.Fb_next[e]; dca = dca + p; }
    const float dfb = dca * a.Ca_prev[e];
    const float dfa = SigmoidDerivOp{}.apply(a.Fb[e], dfb, 0.0f);
    const float zb = a.Zb[e], ib = a.Ib[e];
    const float dib = dca * zb;
    const float dia = SigmoidDerivOp{}.apply(ib, dib, 0.0f);
    const float dzb = dca * ib;
    const float dza = act_backward(act, zb, dzb);
    a.dOb[e] = dob; a.dOa[e] = doa; a.dCb[e] = dcb; a.dCa[e] = dca; a.dFb[e] = dfb; a.dFa[e] = dfa;
    a.dIb[e] = dib; a.dIa[e] = dia; a.dZb[e] = dzb; a.dZa[e] = dza;
    if (PACKED) {
        float* q = a.packed_out + (e / n) * (4 * static_cast<int64_t>(n)) + j;
        q[0] = dza;
        q[n] = dia;
        q[2 * static_cast<int64_t>(n)] = dfa;
        q[3 * static_cast<int64_t>(n)] = doa;
    }
}

}  // namespace bship

namespace bship {
namespace {

int check_step_args(const char* fn, int act, int64_t batch, int64_t n, const void* const* ptrs,
                    int count) {
    if (!ctx().inited)
        return set_error(BSHIP_ERR_NOT_INITIALIZED, "%s: bship_init() has not been called", fn);
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
                          a.dOb, a.dCa, a.dCb, a.pi, a.pf, a.po, a.deltas, a.packed_out};
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

}  // extern "C"
