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

// pool.hip (or a test's stand-in): scratch without zero fill, returned with pool_free_raw
int pool_alloc_raw(size_t nbytes, void** out);
int pool_free_raw(void* p);

namespace window {

// Mode "stacked": the packed copy [dZa|dIa|dFa|dOa] of the gate deltas that the last backward step left behind
// (two buffers that take turns), and the four arrays it is a copy of. Anything else that is enqueued between
// two backward steps may have changed those arrays, so it ends the copy's validity (forget()).
struct PackedDeltas {
    float* buf[2] = {nullptr, nullptr};
    size_t floats = 0;
    int current = 0;
    bool valid = false;
    const char* of[4] = {nullptr, nullptr, nullptr, nullptr};   // dZa, dIa, dFa, dOa
    void forget() { valid = false; }
    int reserve(size_t n) {
        if (n <= floats) return 0;
        release();
        for (int k = 0; k < 2; ++k) {
            void* p = nullptr;
            const int st = pool_alloc_raw(n * sizeof(float), &p);
            if (st != 0) { release(); return st; }
            buf[k] = static_cast<float*>(p);
        }
        floats = n;
        return 0;
    }
    void release() {
        for (int k = 0; k < 2; ++k) {
            if (buf[k]) pool_free_raw(buf[k]);
            buf[k] = nullptr;
        }
        floats = 0;
        valid = false;
    }
};
inline PackedDeltas& packed_deltas() {
    static PackedDeltas state;
    return state;
}

inline const float* cf(const Var& v) { return reinterpret_cast<const float*>(v.p); }
inline float* mf(const Var& v) { return reinterpret_cast<float*>(const_cast<char*>(v.p)); }
inline const float* cf(const char* p) { return reinterpret_cast<const float*>(p); }
inline float* mf(const char* p) { return reinterpret_cast<float*>(const_cast<char*>(p)); }

class DeviceSink : public Sink {
public:
    int primitive(const Rec& r) override {
        packed_deltas().forget();
        switch (r.kind) {
            case K_GEMM:
                return bship_gemm_f32((r.flags & F_TRANSA) ? 1 : 0, (r.flags & F_TRANSB) ? 1 : 0, r.M, r.N, r.K, r.s0,
                                      cf(r.p[0]), r.ld[0], cf(r.p[1]), r.ld[1], r.s1, mf(r.p[2]), r.ld[2]);
            case K_COPY: return bship_d2d(mf(r.p[1]), cf(r.p[0]), r.n * 4);
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

    // lstm_layer.py:117-145 with the four recurrent products as one over [Rz;Ri;Rf;Ro] when the matrices lie
    // back to back (as they do in brainstorm's parameter vector), else as they were called.
    int lstm_forward_with_products(const Match& m, const Rec* q) {
        const Var* v = m.v;
        const size_t square = static_cast<size_t>(m.N) * static_cast<size_t>(m.N) * 4;
        const bool adjacent = v[21].p == v[20].p + square && v[22].p == v[21].p + square && v[23].p == v[22].p + square;
        if (!adjacent) {
            int st = 0;
            for (int k : {0, 3, 7, 13})
                if ((st = primitive(q[k])) != 0) return st;
            return bship_lstm_fwd_step_f32(m.act, m.M, m.N, mf(v[0]), mf(v[1]), mf(v[2]), mf(v[3]), mf(v[4]), mf(v[5]),
                                           mf(v[6]), mf(v[7]), mf(v[8]), mf(v[9]), cf(v[10]), mf(v[11]), cf(v[12]),
                                           cf(v[13]), cf(v[14]), cf(v[15]), cf(v[16]), cf(v[17]), cf(v[18]));
        }
        void* rec = nullptr;
        int st = pool_alloc_raw(static_cast<size_t>(m.M) * static_cast<size_t>(4 * m.N) * sizeof(float), &rec);
        if (st != 0) return st;
        st = bship_gemm_f32(0, 1, m.M, 4 * m.N, m.N, 1.0f, cf(v[19]), m.N, cf(v[20]), m.N, 0.0f,
                            static_cast<float*>(rec), 4 * m.N);
        if (st == 0)
            st = bship_lstm_fwd_step_packed_f32(m.act, m.M, m.N, static_cast<const float*>(rec), mf(v[0]), mf(v[1]),
                                                mf(v[2]), mf(v[3]), mf(v[4]), mf(v[5]), mf(v[6]), mf(v[7]), mf(v[8]),
                                                mf(v[9]), cf(v[10]), mf(v[11]), cf(v[12]), cf(v[13]), cf(v[14]),
                                                cf(v[15]), cf(v[16]), cf(v[17]), cf(v[18]));
        pool_free_raw(rec);       // the block's next owner runs behind these launches
        return st;
    }

    // lstm_layer.py:173-205. With the packed copy of the following step's gate deltas at hand (left by this
    // function when it ran for that step) the four products into dy[t] are one; the step kernel adds deltas[t]
    // and leaves the packed copy of this step's gate deltas for the next call.
    int lstm_backward_with_products(const Match& m, const Rec* q) {
        const Var* v = m.v;
        PackedDeltas& pd = packed_deltas();
        const size_t need = static_cast<size_t>(m.M) * static_cast<size_t>(4 * m.N);
        const bool was_valid = pd.valid && need <= pd.floats;      // new buffers hold nothing yet
        pd.forget();
        int st = pd.reserve(need);
        if (st != 0) return st;
        const size_t square = static_cast<size_t>(m.N) * static_cast<size_t>(m.N) * 4;
        // the weights in the order of the parameter vector: Rz, Ri, Rf, Ro = operands 28, 25, 26, 27
        const bool adjacent = v[25].p == v[28].p + square && v[26].p == v[25].p + square && v[27].p == v[26].p + square;
        // the packed copy holds [dZa|dIa|dFa|dOa] of the step whose arrays are this step's "next" operands
        const bool have = was_valid && adjacent && pd.of[0] == v[30].p && pd.of[1] == v[8].p && pd.of[2] == v[9].p &&
                          pd.of[3] == v[29].p;
        float* out = pd.buf[1 - pd.current];
        if (have) {
            st = bship_gemm_f32(0, 0, m.M, m.N, 4 * m.N, 1.0f, pd.buf[pd.current], 4 * m.N, cf(v[28]), m.N, 0.0f,
                                mf(v[0]), m.N);
        } else {
            for (int k = 0; k < 5 && st == 0; ++k) st = primitive(q[k]);     // the copy and the four products
            pd.forget();
        }
        if (st != 0) return st;
        st = bship_lstm_bwd_step_packed_f32(m.act, m.M, m.N, have ? cf(v[24]) : nullptr, mf(v[0]), out, cf(v[1]),
                                            cf(v[2]), cf(v[3]), cf(v[4]), cf(v[5]), cf(v[6]), cf(v[7]), cf(v[8]),
                                            cf(v[9]), cf(v[10]), mf(v[11]), mf(v[12]), mf(v[13]), mf(v[14]),
                                            mf(v[15]), mf(v[16]), mf(v[17]), mf(v[18]), mf(v[19]), mf(v[20]),
                                            cf(v[21]), cf(v[22]), cf(v[23]));
        if (st != 0) return st;
        pd.current = 1 - pd.current;
        pd.of[0] = v[11].p; pd.of[1] = v[13].p; pd.of[2] = v[15].p; pd.of[3] = v[17].p;
        pd.valid = true;
        return 0;
    }

    int fused(const Pattern& P, const Match& m, const Rec* q) override {
        const Var* v = m.v;
        if (P.id != P_LSTM_BWD_STACKED) packed_deltas().forget();
        switch (P.id) {
            case P_LSTM_FWD_STACKED: return lstm_forward_with_products(m, q);
            case P_LSTM_BWD_STACKED: return lstm_backward_with_products(m, q);
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
