// How the fusing window's decisions become calls of the library's entry points: a held operation
// that is let go is the call it was, a complete sequence is the fused entry point that computes it.
// Kept apart from the library's queue (window.hip) so that a host-only build can route the same
// calls into a trace and check operand orders without a device.
#pragma once

#include "../../include/bship.h"
#include "window_core.h"

namespace bship {

int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int flush_deferred_fills();
int batchnorm_fwd_train_launch(const float* inputs, const float* gamma, const float* beta, float* mu, float* sigma,
                               float* sigma_b, float* centered, float* x_hat, float* out, int64_t M, int64_t N,
                               float neg_inv_m, float decay_mu, float rest_mu, float inv_m, float eps,
                               float decay_sigma, float rest_sigma);

namespace window {

inline const float* cf(const Var& v) { return reinterpret_cast<const float*>(v.p); }
inline float* mf(const Var& v) { return reinterpret_cast<float*>(const_cast<char*>(v.p)); }
inline const float* cf(const char* p) { return reinterpret_cast<const float*>(p); }
inline float* mf(const char* p) { return reinterpret_cast<float*>(const_cast<char*>(p)); }

class DeviceSink : public Sink {
public:
    int primitive(const Rec& r) override {
        switch (r.kind) {
            case K_BINARY: return bship_binary_f32(r.op, cf(r.p[0]), cf(r.p[1]), mf(r.p[2]), r.n);
            case K_MULT_ADD_TT: return bship_mult_add_tt_f32(cf(r.p[0]), cf(r.p[1]), mf(r.p[2]), r.n);
            case K_SCALAR: return bship_scalar_f32(r.op, r.s0, cf(r.p[0]), mf(r.p[1]), r.n);
            case K_UNARY: return bship_unary_f32(r.op, cf(r.p[0]), mf(r.p[1]), r.n);
            case K_DERIV: return bship_deriv_f32(r.op, cf(r.p[0]), cf(r.p[1]), mf(r.p[2]), r.n);
            case K_CLIP: return bship_clip_f32(cf(r.p[0]), r.s0, r.s1, mf(r.p[1]), r.n);
            case K_MV:
                return bship_mv_f32(r.op, cf(r.p[0]), cf(r.p[1]), mf(r.p[2]), r.M, r.N, (r.flags & F_COL) ? 1 : 0,
                                    (r.flags & F_ACC) ? 1 : 0);
            case K_FILL: return bship_fill_f32(mf(r.p[0]), r.s0, r.n);
            case K_SUM: return bship_sum_f32(cf(r.p[0]), mf(r.p[1]), r.M, r.N, r.op);
            case K_SOFTMAX: return bship_softmax_rows_f32(cf(r.p[0]), mf(r.p[1]), r.M, r.N);
            case K_INDEX: return bship_index_m_by_v_f32(cf(r.p[0]), cf(r.p[1]), mf(r.p[2]), r.M, r.N);
            case K_BINARIZE: return bship_binarize_f32(cf(r.p[0]), mf(r.p[1]), r.M, r.N);
            case K_MASK:
                if (r.flags & F_FAST)
                    return r.gen >= 0 ? bship_prob_mask_fast_on_f32(r.gen, mf(r.p[0]), r.n, r.d)
                                      : bship_prob_mask_fast_f32(mf(r.p[0]), r.n, r.d);
                return r.gen >= 0 ? bship_prob_mask_on_f32(r.gen, mf(r.p[0]), r.n, r.d)
                                  : bship_prob_mask_f32(mf(r.p[0]), r.n, r.d);
        }
        return set_error(BSHIP_ERR_BAD_OP, "fusing window: unknown operation kind %d", r.kind);
    }

    int fused(const Pattern& P, const Match& m, const Rec* q) override {
        const Var* v = m.v;
        switch (P.id) {
            case P_LSTM_FWD:
                return bship_lstm_fwd_step_f32(m.act, m.M, m.N, mf(v[0]), mf(v[1]), mf(v[2]), mf(v[3]), mf(v[4]),
                                               mf(v[5]), mf(v[6]), mf(v[7]), mf(v[8]), mf(v[9]), cf(v[10]), mf(v[11]),
                                               cf(v[12]), cf(v[13]), cf(v[14]), cf(v[15]), cf(v[16]), cf(v[17]),
                                               cf(v[18]));
            case P_LSTM_BWD:
                return bship_lstm_bwd_step_f32(m.act, m.M, m.N, cf(v[0]), cf(v[1]), cf(v[2]), cf(v[3]), cf(v[4]),
                                               cf(v[5]), cf(v[6]), cf(v[7]), cf(v[8]), cf(v[9]), cf(v[10]), mf(v[11]),
                                               mf(v[12]), mf(v[13]), mf(v[14]), mf(v[15]), mf(v[16]), mf(v[17]),
                                               mf(v[18]), mf(v[19]), mf(v[20]), cf(v[21]), cf(v[22]), cf(v[23]));
            case P_BIAS_ACT:
                return bship_bias_act_f32(m.act, cf(v[0]), cf(v[1]), mf(v[2]), m.M, m.N);
            case P_DROPOUT: {
                const Rec& mask = q[0];
                const size_t n = static_cast<size_t>(m.total);
                if (mask.flags & F_FAST)
                    return mask.gen >= 0
                               ? bship_dropout_fwd_fast_on_f32(mask.gen, cf(v[1]), mf(v[0]), mf(v[2]), n, mask.d, q[2].s0)
                               : bship_dropout_fwd_fast_f32(cf(v[1]), mf(v[0]), mf(v[2]), n, mask.d, q[2].s0);
                return mask.gen >= 0 ? bship_dropout_fwd_on_f32(mask.gen, cf(v[1]), mf(v[0]), mf(v[2]), n, mask.d, q[2].s0)
                                     : bship_dropout_fwd_f32(cf(v[1]), mf(v[0]), mf(v[2]), n, mask.d, q[2].s0);
            }
            case P_SOFTMAX_CE_FWD:
                return bship_softmax_ce_fwd_f32(cf(v[0]), cf(v[3]), mf(v[1]), mf(v[2]), m.M, m.N);
            case P_SOFTMAX_CE_BWD:
                return bship_softmax_ce_bwd_f32(cf(v[2]), cf(v[0]), cf(v[3]), mf(v[1]), mf(v[4]), m.M, m.N);
            case P_MOMENTUM:
                return bship_momentum_update_f32(q[0].s0, q[1].s0, cf(v[1]), mf(v[0]), mf(v[2]),
                                                 static_cast<size_t>(m.total));
            case P_HIGHWAY_FWD:
                return bship_highway_fwd_f32(cf(v[0]), cf(v[3]), cf(v[1]), mf(v[4]), static_cast<size_t>(m.total));
            case P_HIGHWAY_BWD:
                return bship_highway_bwd_f32(cf(v[5]), cf(v[1]), cf(v[6]), cf(v[2]), mf(v[3]), mf(v[4]), mf(v[7]),
                                             static_cast<size_t>(m.total));
            case P_BN_FWD: {
                const int st = flush_deferred_fills();      // an internal launcher: the entry points do this themselves
                if (st != 0) return st;
                return batchnorm_fwd_train_launch(cf(v[0]), cf(v[6]), cf(v[8]), mf(v[2]), mf(v[5]), mf(v[1]), mf(v[3]),
                                                  mf(v[4]), mf(v[7]), m.M, m.N, q[1].s0, q[2].s0, q[3].s0, q[7].s0,
                                                  q[8].s0, q[10].s0, q[11].s0);
            }
            case P_BN_INFER:
                return bship_batchnorm_fwd_f32(0, cf(v[0]), cf(v[5]), cf(v[7]), mf(v[1]), mf(v[3]), 0.0, 0.0, mf(v[3]),
                                               mf(v[2]), mf(v[4]), mf(v[6]), m.M, m.N);
            case P_BN_BWD:
                return bship_batchnorm_bwd_f32(cf(v[0]), cf(v[1]), cf(v[6]), cf(v[7]), mf(v[4]), mf(v[5]), mf(v[8]),
                                               m.M, m.N);
        }
        return set_error(BSHIP_ERR_BAD_OP, "fusing window: unknown sequence %d", P.id);
    }
};

}  // namespace window
}  // namespace bship
