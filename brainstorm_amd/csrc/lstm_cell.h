// The elementwise part of one LSTM forward time step for one element (lstm_layer.py:117-145), shared by
// the per-step kernels (fused.hip) and the whole-sequence kernel (lstm_seq.hip) so that both apply the
// same float32 operations in the same order as the layer's primitive calls:
//   add_mv(Za, bz); Zb = act(Za)
//   mult_add_mv(Ca_prev, pi, Ia); add_mv(Ia, bi); Ib = sigmoid(Ia)
//   mult_add_mv(Ca_prev, pf, Fa); add_mv(Fa, bf); Fb = sigmoid(Fa)
//   Ca = Ib * Zb; mult_add_tt(Fb, Ca_prev, Ca)
//   mult_add_mv(Ca, po, Oa); add_mv(Oa, bo); Ob = sigmoid(Oa)
//   Cb = act(Ca); y = Ob * Cb
#pragma once
#pragma clang fp contract(off)

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

// In: za, ia, fa, oa with the input and recurrent products accumulated. Out: everything the layer keeps.
struct LstmCell {
    float za, zb, ia, ib, fa, fb, oa, ob, ca, cb, y;
};

__device__ __forceinline__ void lstm_cell_forward(LstmCell& c, int act, float c_prev, float pi, float pf, float po,
                                                  float bz, float bi, float bf, float bo) {
    c.za = c.za + bz;
    c.zb = act_forward(act, c.za);
    { const float p = c_prev * pi; c.ia = c.ia + p; }
    c.ia = c.ia + bi;
    c.ib = SigmoidOp{}.apply(c.ia, 0.0f, 0.0f);
    { const float p = c_prev * pf; c.fa = c.fa + p; }
    c.fa = c.fa + bf;
    c.fb = SigmoidOp{}.apply(c.fa, 0.0f, 0.0f);
    c.ca = c.ib * c.zb;
    { const float p = c.fb * c_prev; c.ca = c.ca + p; }
    { const float p = c.ca * po; c.oa = c.oa + p; }
    c.oa = c.oa + bo;
    c.ob = SigmoidOp{}.apply(c.oa, 0.0f, 0.0f);
    c.cb = act_forward(act, c.ca);
    c.y = c.ob * c.cb;
}

}  // namespace bship
