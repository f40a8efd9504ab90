// The fusing window: a short queue of handler operations that have been asked for but not yet
// enqueued on the device, and the matcher that recognises in it the operation sequences of
// brainstorm's layers, so that a caller who only knows the primitive handler interface gets
// the fused kernels.
//
// A brainstorm layer is a fixed sequence of handler calls on views of the network's buffers
// (layers/lstm_layer.py:115-145 and 167-205, batch_normalization_layer.py:68-152,
// highway_layer.py:40-71, fully_connected_layer.py:52-64, dropout_layer.py:36-45,
// softmax_ce_layer.py:65-114, training/steppers.py:97-114). Each such sequence is written down
// below as a pattern: operation kinds and codes, and which operand of which call is the same
// array as which operand of another call (by address and length). Calls are held back only
// while they are a prefix of some pattern; a complete pattern is replaced by one fused launch
// whose kernel chains the same float32 functors in the same order (same bits); anything else
// is enqueued as it is, in call order.
//
// Temporaries. Some layers compute through arrays they allocate and drop (highway_layer.py:48,
// 64; batch_normalization_layer.py:119-120). Their fused kernels do not write those arrays, so
// the fused launch is only taken when the temporaries are returned to the pool right behind
// the last call of the pattern (which is what dropping the last reference does); any other
// call first enqueues the held operations unfused.
//
// Matrix products are not held: they pass the window and may overtake the held operations when
// they touch none of their operands (the four recurrent products of an LSTM time step lie
// between elementwise calls that work on other arrays).
//
// This header is plain C++ (no device code) so that the matcher can be exercised on the host.
#pragma once

#include <stddef.h>
#include <stdint.h>
#include <string.h>

namespace bship {
namespace window {

enum Kind : uint8_t {
    K_BINARY,       // p0 = a, p1 = b, p2 = out; op = BSHIP_ADD ...
    K_MULT_ADD_TT,  // p0 = a, p1 = b, p2 = out (read and written)
    K_SCALAR,       // p0 = t, p1 = out; op = BSHIP_ADD_ST ...; s0 = scalar
    K_UNARY,        // p0 = x, p1 = y; op = BSHIP_ABS ...
    K_DERIV,        // p0 = y, p1 = dy, p2 = dx; op = BSHIP_SIGMOID_DERIV ...
    K_CLIP,         // p0 = a, p1 = out; s0 = low, s1 = high
    K_MV,           // p0 = m, p1 = v, p2 = out; op = BSHIP_ADD ...; flags F_COL, F_ACC; M, N
    K_FILL,         // p0 = mem; s0 = value
    K_SUM,          // p0 = a, p1 = out; op = axis (0, 1, -1); M, N
    K_SOFTMAX,      // p0 = m, p1 = out; M, N
    K_INDEX,        // p0 = m, p1 = v, p2 = out; M, N (= K columns)
    K_BINARIZE,     // p0 = v, p1 = out; M, N (= K columns)
    K_MASK,         // p0 = mask; d = probability; gen = generator; flags F_FAST
    K_GEMM,         // p0 = A, p1 = B, p2 = C; flags F_TRANSA, F_TRANSB; M, N, K, ld[]; s0 = alpha, s1 = beta
    K_COPY,         // p0 = source, p1 = destination; n elements
    K_KINDS
};

enum : uint8_t { F_COL = 1, F_ACC = 2, F_FAST = 1, F_TRANSA = 1, F_TRANSB = 2 };

// operation codes of include/bship.h that the patterns name
enum { OP_ADD = 0, OP_SUB = 1, OP_MUL = 2, OP_DIV = 3 };
enum { OP_ADD_ST = 0, OP_MULT_ST = 1, OP_MULT_ADD_ST = 2 };
enum { OP_SQRT = 2, OP_LOG = 3, OP_SIGMOID = 4, OP_TANH = 5, OP_REL = 6, OP_EL = 7 };
enum { OP_SIGMOID_DERIV = 0, OP_TANH_DERIV = 1, OP_REL_DERIV = 2, OP_EL_DERIV = 3 };
// activation codes of the fused entry points (lstm_cell.h)
enum { ACT_SIGMOID = 0, ACT_TANH = 1, ACT_REL = 2, ACT_LINEAR = 3, ACT_EL = 4 };

constexpr int kMaxPtrs = 3;

struct Rec {
    uint8_t kind = 0;
    int8_t op = 0;
    uint8_t flags = 0;
    uint8_t nptr = 0;
    uint8_t rd = 0, wr = 0;            // bit s: operand s is read / written
    const char* p[kMaxPtrs] = {nullptr, nullptr, nullptr};
    size_t len[kMaxPtrs] = {0, 0, 0};  // bytes
    size_t n = 0;                      // elements of the elementwise kinds
    int64_t M = 0, N = 0;              // rows and columns of the matrix kinds
    int64_t K = 0, ld[kMaxPtrs] = {0, 0, 0};   // matrix products: inner dimension, row pitches of A, B, C
    float s0 = 0.0f, s1 = 0.0f;
    double d = 0.0;
    int gen = 0;
};

inline void set_ptr(Rec& r, int s, const void* p, size_t bytes, bool read, bool written) {
    r.p[s] = static_cast<const char*>(p);
    r.len[s] = bytes;
    if (read) r.rd |= uint8_t(1u << s);
    if (written) r.wr |= uint8_t(1u << s);
    if (s + 1 > r.nptr) r.nptr = uint8_t(s + 1);
}

inline Rec rec_binary(int op, const void* a, const void* b, void* out, size_t n) {
    Rec r; r.kind = K_BINARY; r.op = int8_t(op); r.n = n;
    set_ptr(r, 0, a, n * 4, true, false); set_ptr(r, 1, b, n * 4, true, false); set_ptr(r, 2, out, n * 4, false, true);
    return r;
}
inline Rec rec_mult_add_tt(const void* a, const void* b, void* out, size_t n) {
    Rec r; r.kind = K_MULT_ADD_TT; r.n = n;
    set_ptr(r, 0, a, n * 4, true, false); set_ptr(r, 1, b, n * 4, true, false); set_ptr(r, 2, out, n * 4, true, true);
    return r;
}
inline Rec rec_scalar(int op, float s, const void* t, void* out, size_t n) {
    Rec r; r.kind = K_SCALAR; r.op = int8_t(op); r.n = n; r.s0 = s;
    set_ptr(r, 0, t, n * 4, true, false); set_ptr(r, 1, out, n * 4, op == OP_MULT_ADD_ST, true);
    return r;
}
inline Rec rec_unary(int op, const void* x, void* y, size_t n) {
    Rec r; r.kind = K_UNARY; r.op = int8_t(op); r.n = n;
    set_ptr(r, 0, x, n * 4, true, false); set_ptr(r, 1, y, n * 4, false, true);
    return r;
}
inline Rec rec_deriv(int op, const void* y, const void* dy, void* dx, size_t n) {
    Rec r; r.kind = K_DERIV; r.op = int8_t(op); r.n = n;
    set_ptr(r, 0, y, n * 4, true, false); set_ptr(r, 1, dy, n * 4, true, false); set_ptr(r, 2, dx, n * 4, false, true);
    return r;
}
inline Rec rec_clip(const void* a, float lo, float hi, void* out, size_t n) {
    Rec r; r.kind = K_CLIP; r.n = n; r.s0 = lo; r.s1 = hi;
    set_ptr(r, 0, a, n * 4, true, false); set_ptr(r, 1, out, n * 4, false, true);
    return r;
}
inline Rec rec_mv(int op, const void* m, const void* v, void* out, int64_t M, int64_t N, bool col, bool acc) {
    Rec r; r.kind = K_MV; r.op = int8_t(op); r.M = M; r.N = N; r.n = size_t(M) * size_t(N);
    r.flags = uint8_t((col ? F_COL : 0) | (acc ? F_ACC : 0));
    set_ptr(r, 0, m, r.n * 4, true, false); set_ptr(r, 1, v, size_t(col ? M : N) * 4, true, false);
    set_ptr(r, 2, out, r.n * 4, acc, true);
    return r;
}
inline Rec rec_fill(void* mem, float val, size_t n) {
    Rec r; r.kind = K_FILL; r.n = n; r.s0 = val;
    set_ptr(r, 0, mem, n * 4, false, true);
    return r;
}
inline Rec rec_sum(const void* a, void* out, int64_t M, int64_t N, int axis) {
    Rec r; r.kind = K_SUM; r.op = int8_t(axis); r.M = M; r.N = N; r.n = size_t(M) * size_t(N);
    set_ptr(r, 0, a, r.n * 4, true, false);
    set_ptr(r, 1, out, size_t(axis == 0 ? N : (axis == 1 ? M : 1)) * 4, false, true);
    return r;
}
inline Rec rec_softmax(const void* m, void* out, int64_t M, int64_t N) {
    Rec r; r.kind = K_SOFTMAX; r.M = M; r.N = N; r.n = size_t(M) * size_t(N);
    set_ptr(r, 0, m, r.n * 4, true, false); set_ptr(r, 1, out, r.n * 4, false, true);
    return r;
}
inline Rec rec_index(const void* m, const void* v, void* out, int64_t M, int64_t K) {
    Rec r; r.kind = K_INDEX; r.M = M; r.N = K; r.n = size_t(M) * size_t(K);
    set_ptr(r, 0, m, r.n * 4, true, false); set_ptr(r, 1, v, size_t(M) * 4, true, false);
    set_ptr(r, 2, out, size_t(M) * 4, false, true);
    return r;
}
inline Rec rec_binarize(const void* v, void* out, int64_t M, int64_t K) {
    Rec r; r.kind = K_BINARIZE; r.M = M; r.N = K; r.n = size_t(M) * size_t(K);
    set_ptr(r, 0, v, size_t(M) * 4, true, false); set_ptr(r, 1, out, r.n * 4, false, true);
    return r;
}
inline Rec rec_mask(void* mask, size_t n, double p, int gen, bool fast) {
    Rec r; r.kind = K_MASK; r.n = n; r.d = p; r.gen = gen; r.flags = fast ? F_FAST : 0;
    set_ptr(r, 0, mask, n * 4, false, true);
    return r;
}

inline Rec rec_gemm(bool transa, bool transb, int64_t M, int64_t N, int64_t K, float alpha, const void* A, int64_t lda,
                    const void* B, int64_t ldb, float beta, void* C, int64_t ldc) {
    Rec r; r.kind = K_GEMM; r.M = M; r.N = N; r.K = K; r.n = size_t(M) * size_t(N); r.s0 = alpha; r.s1 = beta;
    r.flags = uint8_t((transa ? F_TRANSA : 0) | (transb ? F_TRANSB : 0));
    r.ld[0] = lda; r.ld[1] = ldb; r.ld[2] = ldc;
    const int64_t a_rows = transa ? K : M, a_cols = transa ? M : K, b_rows = transb ? N : K, b_cols = transb ? K : N;
    set_ptr(r, 0, A, size_t((a_rows - 1) * lda + a_cols) * 4, true, false);
    set_ptr(r, 1, B, size_t((b_rows - 1) * ldb + b_cols) * 4, true, false);
    set_ptr(r, 2, C, size_t((M - 1) * ldc + N) * 4, beta != 0.0f, true);
    return r;
}
inline Rec rec_copy(const void* src, void* dst, size_t n) {
    Rec r; r.kind = K_COPY; r.n = n;
    set_ptr(r, 0, src, n * 4, true, false); set_ptr(r, 1, dst, n * 4, false, true);
    return r;
}

// ------------------------------------------------------------------ patterns
enum PatternId {
    P_LSTM_FWD, P_LSTM_BWD, P_BIAS_ACT, P_DROPOUT, P_SOFTMAX_CE_FWD, P_SOFTMAX_CE_BWD, P_MOMENTUM,
    P_HIGHWAY_FWD, P_HIGHWAY_BWD, P_BN_FWD, P_BN_INFER, P_BN_BWD,
    // with matrix products held as well (mode "stacked"): a whole LSTM time step including its four
    // recurrent products, which then run as one product over the stacked matrices
    P_LSTM_FWD_STACKED, P_LSTM_BWD_STACKED, P_COUNT
};
constexpr int kPlainPatterns = P_LSTM_FWD_STACKED;     // the patterns of the same-bits mode come first

enum : int8_t { OP_ANY_ACT = -2, OP_ANY_ACT_DERIV = -3 };   // an activation; the same one throughout a pattern
enum Size : uint8_t { S_MN, S_M, S_N };                       // elements of an elementwise call: M*N, M or N
enum Check : uint8_t { C_NONE, C_ONE, C_MINUS_ONE, C_CE_CLIP };   // s0 == 1 / s0 == -1 / clip to [1e-6, 1]

struct Elem {
    uint8_t kind;
    int8_t op;
    uint8_t flags;
    int8_t v[kMaxPtrs];   // the pattern's variable behind each operand
    uint8_t size;
    uint8_t check;
};

constexpr int kMaxVars = 32;
constexpr int kMaxElems = 20;

struct Pattern {
    int id;
    const char* name;
    int len;
    Elem e[kMaxElems];
    int ntemps;            // variables that the fused kernel does not write: must have been freed
    int8_t temps[2];
    int8_t alias[2];       // one pair of variables that may be the same array exactly (in-place form), or -1
};

#define W_E(kind, op, flags, a, b, c, size, check) {kind, int8_t(op), flags, {a, b, c}, size, check}

inline const Pattern* patterns() {
    static const Pattern table[P_COUNT] = {
        // lstm_layer.py:121-145 without its four dot_add_mm (they pass the window).
        // Za0 Zb1 Ia2 Ib3 Fa4 Fb5 Oa6 Ob7 Ca8 Cb9 Cprev10 y11 pi12 pf13 po14 bz15 bi16 bf17 bo18
        {P_LSTM_FWD, "lstm_forward_step", 15,
         {W_E(K_MV, OP_ADD, 0, 0, 15, 0, S_MN, C_NONE),
          W_E(K_UNARY, OP_ANY_ACT, 0, 0, 1, -1, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 10, 12, 2, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 2, 16, 2, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 2, 3, -1, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 10, 13, 4, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 4, 17, 4, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 4, 5, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 3, 1, 8, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 5, 10, 8, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 8, 14, 6, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 6, 18, 6, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 6, 7, -1, S_MN, C_NONE),
          W_E(K_UNARY, OP_ANY_ACT, 0, 8, 9, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 7, 9, 11, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // lstm_layer.py:180-205 behind copy_to and the four dot_add_mm into dy[t].
        // dy0 Zb1 Ib2 Fb3 Ob4 Cb5 Cprev6 Fbn7 dIan8 dFan9 dCan10 dZa11 dZb12 dIa13 dIb14 dFa15 dFb16
        // dOa17 dOb18 dCa19 dCb20 pi21 pf22 po23
        {P_LSTM_BWD, "lstm_backward_step", 15,
         {W_E(K_MV, OP_MUL, F_ACC, 8, 21, 19, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 9, 22, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 0, 5, 18, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 4, 18, 17, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 17, 23, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 0, 4, 20, S_MN, C_NONE),
          W_E(K_DERIV, OP_ANY_ACT_DERIV, 0, 5, 20, 20, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 19, 20, 19, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 10, 7, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 6, 16, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 3, 16, 15, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 1, 14, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 2, 14, 13, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 2, 12, S_MN, C_NONE),
          W_E(K_DERIV, OP_ANY_ACT_DERIV, 0, 1, 12, 11, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // fully_connected_layer.py:61-62: add_mv(m, bias, out); act(out, out).  m0 bias1 out2
        {P_BIAS_ACT, "bias_act", 2,
         {W_E(K_MV, OP_ADD, 0, 0, 1, 2, S_MN, C_NONE),
          W_E(K_UNARY, OP_ANY_ACT, 0, 2, 2, -1, S_MN, C_NONE)},
         0, {-1, -1}, {0, 2}},
        // dropout_layer.py:41-45.  mask0 in1 out2
        {P_DROPOUT, "dropout_forward", 3,
         {W_E(K_MASK, 0, 0, 0, -1, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 1, 0, 2, S_MN, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 2, 2, -1, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // softmax_ce_layer.py:79-89.  in0 probs1 loss2 targets3
        {P_SOFTMAX_CE_FWD, "softmax_ce_forward", 6,
         {W_E(K_SOFTMAX, 0, 0, 0, 1, -1, S_MN, C_NONE),
          W_E(K_FILL, 0, 0, 2, -1, -1, S_M, C_NONE),
          W_E(K_INDEX, 0, 0, 1, 3, 2, S_MN, C_NONE),
          W_E(K_CLIP, 0, 0, 2, 2, -1, S_M, C_CE_CLIP),
          W_E(K_UNARY, OP_LOG, 0, 2, 2, -1, S_M, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 2, 2, -1, S_M, C_MINUS_ONE)},
         0, {-1, -1}, {-1, -1}},
        // softmax_ce_layer.py:108-112.  targets0 t_bin1 probs2 dloss3 dinputs4
        {P_SOFTMAX_CE_BWD, "softmax_ce_backward", 5,
         {W_E(K_BINARIZE, 0, 0, 0, 1, -1, S_MN, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 1, 1, -1, S_MN, C_MINUS_ONE),
          W_E(K_BINARY, OP_ADD, 0, 1, 2, 1, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_COL, 1, 3, 1, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 1, 4, 4, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // steppers.py:104-112.  velocity0 gradients1 parameters2
        {P_MOMENTUM, "momentum_update", 3,
         {W_E(K_SCALAR, OP_MULT_ST, 0, 0, 0, -1, S_MN, C_NONE),
          W_E(K_SCALAR, OP_MULT_ADD_ST, 0, 1, 0, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 0, 2, 2, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // highway_layer.py:48-51.  H0 x1 tmp2 T3 y4
        {P_HIGHWAY_FWD, "highway_forward", 3,
         {W_E(K_BINARY, OP_SUB, 0, 0, 1, 2, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 3, 2, 2, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 2, 1, 4, S_MN, C_NONE)},
         1, {2, -1}, {-1, -1}},
        // highway_layer.py:64-71 (ones = fill with 1).  tmp0 T1 dy2 dx3 dH4 H5 x6 dT7
        {P_HIGHWAY_BWD, "highway_backward", 6,
         {W_E(K_FILL, 0, 0, 0, -1, -1, S_MN, C_ONE),
          W_E(K_BINARY, OP_SUB, 0, 0, 1, 0, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 0, 2, 3, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 1, 2, 4, S_MN, C_NONE),
          W_E(K_BINARY, OP_SUB, 0, 5, 6, 0, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 0, 2, 7, S_MN, C_NONE)},
         1, {0, -1}, {-1, -1}},
        // batch_normalization_layer.py:68-105, training.
        // in0 sigma_b1 mu2 centered3 x_hat4 sigma5 gamma6 out7 beta8
        {P_BN_FWD, "batchnorm_forward", 15,
         {W_E(K_SUM, 0, 0, 0, 1, -1, S_MN, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 1, 1, -1, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 2, 2, -1, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ADD_ST, 0, 1, 2, -1, S_N, C_NONE),
          W_E(K_MV, OP_ADD, 0, 0, 1, 3, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 3, 3, 4, S_MN, C_NONE),
          W_E(K_SUM, 0, 0, 4, 1, -1, S_MN, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 1, 1, -1, S_N, C_NONE),
          W_E(K_SCALAR, OP_ADD_ST, 0, 1, 1, -1, S_N, C_NONE),
          W_E(K_UNARY, OP_SQRT, 0, 1, 1, -1, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 5, 5, -1, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ADD_ST, 0, 1, 5, -1, S_N, C_NONE),
          W_E(K_MV, OP_DIV, 0, 3, 1, 4, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, 0, 4, 6, 7, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 7, 8, 7, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // batch_normalization_layer.py:79-105 with the running statistics (no training pass).
        // in0 mu1 centered2 sigma3 x_hat4 gamma5 out6 beta7
        {P_BN_INFER, "batchnorm_inference", 4,
         {W_E(K_MV, OP_ADD, 0, 0, 1, 2, S_MN, C_NONE),
          W_E(K_MV, OP_DIV, 0, 2, 3, 4, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, 0, 4, 5, 6, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 6, 7, 6, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // batch_normalization_layer.py:119-152.
        // dout0 x_hat1 big2 small3 dgamma4 dbeta5 gamma6 sigma_b7 din8
        {P_BN_BWD, "batchnorm_backward", 13,
         {W_E(K_BINARY, OP_MUL, 0, 0, 1, 2, S_MN, C_NONE),
          W_E(K_SUM, 0, 0, 2, 3, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 3, 4, 4, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 3, 3, -1, S_N, C_NONE),
          W_E(K_MV, OP_MUL, 0, 1, 3, 2, S_MN, C_NONE),
          W_E(K_SUM, 0, 0, 0, 3, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 3, 5, 5, S_N, C_NONE),
          W_E(K_SCALAR, OP_MULT_ST, 0, 3, 3, -1, S_N, C_NONE),
          W_E(K_BINARY, OP_SUB, 0, 0, 2, 2, S_MN, C_NONE),
          W_E(K_MV, OP_SUB, 0, 2, 3, 2, S_MN, C_NONE),
          W_E(K_BINARY, OP_DIV, 0, 6, 7, 3, S_N, C_NONE),
          W_E(K_MV, OP_MUL, 0, 2, 3, 2, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 2, 8, 8, S_MN, C_NONE)},
         2, {2, 3}, {-1, -1}},
        // lstm_layer.py:121-145 with its four dot_add_mm(y[t-1], R*, *a[t], transb=True).
        // operands 0-18 as in lstm_forward_step; yprev19 Rz20 Ri21 Rf22 Ro23
        {P_LSTM_FWD_STACKED, "lstm_forward_step_with_products", 19,
         {W_E(K_GEMM, 0, F_TRANSB, 19, 20, 0, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 0, 15, 0, S_MN, C_NONE),
          W_E(K_UNARY, OP_ANY_ACT, 0, 0, 1, -1, S_MN, C_NONE),
          W_E(K_GEMM, 0, F_TRANSB, 19, 21, 2, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 10, 12, 2, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 2, 16, 2, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 2, 3, -1, S_MN, C_NONE),
          W_E(K_GEMM, 0, F_TRANSB, 19, 22, 4, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 10, 13, 4, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 4, 17, 4, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 4, 5, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 3, 1, 8, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 5, 10, 8, S_MN, C_NONE),
          W_E(K_GEMM, 0, F_TRANSB, 19, 23, 6, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 8, 14, 6, S_MN, C_NONE),
          W_E(K_MV, OP_ADD, 0, 6, 18, 6, S_MN, C_NONE),
          W_E(K_UNARY, OP_SIGMOID, 0, 6, 7, -1, S_MN, C_NONE),
          W_E(K_UNARY, OP_ANY_ACT, 0, 8, 9, -1, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 7, 9, 11, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
        // lstm_layer.py:173-205: copy_to(deltas[t], dy[t]), the four dot_add_mm into dy[t], the elementwise part.
        // operands 0-23 as in lstm_backward_step; deltas24 Ri25 Rf26 Ro27 Rz28 dOan29 dZan30
        {P_LSTM_BWD_STACKED, "lstm_backward_step_with_products", 20,
         {W_E(K_COPY, 0, 0, 24, 0, -1, S_MN, C_NONE),
          W_E(K_GEMM, 0, 0, 8, 25, 0, S_MN, C_NONE),
          W_E(K_GEMM, 0, 0, 9, 26, 0, S_MN, C_NONE),
          W_E(K_GEMM, 0, 0, 29, 27, 0, S_MN, C_NONE),
          W_E(K_GEMM, 0, 0, 30, 28, 0, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 8, 21, 19, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 9, 22, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 0, 5, 18, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 4, 18, 17, S_MN, C_NONE),
          W_E(K_MV, OP_MUL, F_ACC, 17, 23, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 0, 4, 20, S_MN, C_NONE),
          W_E(K_DERIV, OP_ANY_ACT_DERIV, 0, 5, 20, 20, S_MN, C_NONE),
          W_E(K_BINARY, OP_ADD, 0, 19, 20, 19, S_MN, C_NONE),
          W_E(K_MULT_ADD_TT, 0, 0, 10, 7, 19, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 6, 16, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 3, 16, 15, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 1, 14, S_MN, C_NONE),
          W_E(K_DERIV, OP_SIGMOID_DERIV, 0, 2, 14, 13, S_MN, C_NONE),
          W_E(K_BINARY, OP_MUL, 0, 19, 2, 12, S_MN, C_NONE),
          W_E(K_DERIV, OP_ANY_ACT_DERIV, 0, 1, 12, 11, S_MN, C_NONE)},
         0, {-1, -1}, {-1, -1}},
    };
    return table;
}
#undef W_E

struct Var {
    const char* p = nullptr;
    size_t len = 0;
    bool bound = false, written = false;
};

struct Match {
    Var v[kMaxVars];
    int64_t M = -1, N = -1, total = -1;
    int act = -1;
};

inline int act_of_unary(int op) {
    switch (op) {
        case OP_SIGMOID: return ACT_SIGMOID;
        case OP_TANH: return ACT_TANH;
        case OP_REL: return ACT_REL;
        case OP_EL: return ACT_EL;
    }
    return -1;
}
inline int act_of_deriv(int op) {
    switch (op) {
        case OP_SIGMOID_DERIV: return ACT_SIGMOID;
        case OP_TANH_DERIV: return ACT_TANH;
        case OP_REL_DERIV: return ACT_REL;
        case OP_EL_DERIV: return ACT_EL;
    }
    return -1;
}

inline bool has_shape(uint8_t kind) {
    return kind == K_MV || kind == K_SUM || kind == K_SOFTMAX || kind == K_INDEX || kind == K_BINARIZE || kind == K_GEMM;
}

inline bool ranges_overlap(const char* a, size_t alen, const char* b, size_t blen) {
    return alen != 0 && blen != 0 && a < b + blen && b < a + alen;
}

// Does call r agree with element i of the pattern, given the operands met so far (m)? Binds the
// operands it meets for the first time.
inline bool match_call(const Pattern& P, int i, const Rec& r, Match& m) {
    const Elem& e = P.e[i];
    if (r.kind != e.kind) return false;
    if (e.op == OP_ANY_ACT || e.op == OP_ANY_ACT_DERIV) {
        const int a = e.op == OP_ANY_ACT ? act_of_unary(r.op) : act_of_deriv(r.op);
        if (a < 0) return false;
        if (m.act < 0) m.act = a;
        else if (m.act != a) return false;
    } else if (e.kind != K_MASK && e.kind != K_FILL && e.kind != K_CLIP && e.kind != K_MULT_ADD_TT &&
               e.kind != K_SOFTMAX && e.kind != K_INDEX && e.kind != K_BINARIZE && e.kind != K_GEMM && e.kind != K_COPY) {
        if (r.op != e.op) return false;
    }
    if ((e.kind == K_MV || e.kind == K_GEMM) && r.flags != e.flags) return false;
    if (e.kind == K_GEMM) {
        // a recurrent product of an LSTM layer: square weights, dense operands, accumulated into its result
        if (r.s0 != 1.0f || r.s1 != 1.0f || r.K != r.N || r.ld[0] != r.K || r.ld[1] != r.K || r.ld[2] != r.N) return false;
    }
    switch (e.check) {
        case C_ONE: if (r.s0 != 1.0f) return false; break;
        case C_MINUS_ONE: if (r.s0 != -1.0f) return false; break;
        case C_CE_CLIP: if (r.s0 != 1e-6f || r.s1 != 1.0f) return false; break;
        default: break;
    }
    if (has_shape(e.kind)) {
        if (m.M < 0) {
            if (m.total >= 0 && r.M * r.N != m.total) return false;
            m.M = r.M; m.N = r.N; m.total = r.M * r.N;
        } else if (r.M != m.M || r.N != m.N) {
            return false;
        }
    } else {
        int64_t want = e.size == S_MN ? m.total : (e.size == S_M ? m.M : m.N);
        if (want < 0) {
            if (e.size != S_MN) return false;
            m.total = want = static_cast<int64_t>(r.n);
        }
        if (static_cast<int64_t>(r.n) != want) return false;
    }
    for (int s = 0; s < r.nptr; ++s) {
        const int id = e.v[s];
        if (id < 0) return false;
        Var& v = m.v[id];
        if (!v.bound) {
            v.p = r.p[s]; v.len = r.len[s]; v.bound = true;
        } else if (v.p != r.p[s] || v.len != r.len[s]) {
            return false;
        }
        if ((r.wr >> s) & 1) v.written = true;
    }
    return true;
}

// How many of the first min(count, P.len) queued calls agree with the pattern: that number if all
// of them do (m then holds the operands met so far), else -1.
inline int match_prefix(const Pattern& P, const Rec* q, int count, Match& m) {
    m = Match();
    const int k = count < P.len ? count : P.len;
    for (int i = 0; i < k; ++i)
        if (!match_call(P, i, q[i], m)) return -1;
    return k;
}

// Operands that the pattern treats as different arrays must not share memory when one of them is
// written (the fused kernel reads everything of an element first and writes afterwards, the
// separate kernels do not). One pair per pattern may be exactly the same array (in-place form).
inline bool operands_distinct(const Pattern& P, const Match& m) {
    for (int i = 0; i < kMaxVars; ++i) {
        if (!m.v[i].bound) continue;
        for (int j = i + 1; j < kMaxVars; ++j) {
            if (!m.v[j].bound || !(m.v[i].written || m.v[j].written)) continue;
            if (!ranges_overlap(m.v[i].p, m.v[i].len, m.v[j].p, m.v[j].len)) continue;
            const bool pair = (P.alias[0] == i && P.alias[1] == j) || (P.alias[0] == j && P.alias[1] == i);
            if (pair && m.v[i].p == m.v[j].p && m.v[i].len == m.v[j].len) continue;
            return false;
        }
    }
    return true;
}

// What the fused kernel cannot express although the calls line up.
inline bool fusable(const Pattern& P, const Match& m, const Rec* q) {
    if (!operands_distinct(P, m)) return false;
    if (m.total <= 0) return false;
    switch (P.id) {
        case P_BN_BWD: return q[3].s0 == q[7].s0 && m.M >= 1;     // one 1/m for both statistics
        case P_BN_FWD: return m.M >= 1;
        case P_LSTM_FWD: case P_LSTM_BWD: case P_LSTM_FWD_STACKED: case P_LSTM_BWD_STACKED: return m.N <= 0x3fffffff;
        default: return true;
    }
}

struct Stats {
    uint64_t calls = 0;       // operations that entered the window
    uint64_t unfused = 0;     // of those, enqueued as they were
    uint64_t fused_calls = 0; // of those, replaced by fused launches
    uint64_t fused = 0;       // fused launches
    uint64_t overtaken = 0;   // matrix products that passed held operations
    uint64_t per_pattern[P_COUNT] = {0};
};

// Where the window's decisions go: the library enqueues kernels, a test records names.
struct Sink {
    virtual int primitive(const Rec& r) = 0;
    virtual int fused(const Pattern& P, const Match& m, const Rec* q) = 0;
    virtual ~Sink() {}
};

constexpr int kQueue = 32;

class Matcher {
public:
    int held() const { return count_; }
    // With `stacked`, the patterns that hold matrix products are in play as well (the caller then hands
    // products and copies to push() instead of letting them pass).
    void set_stacked(bool on) { npatterns_ = on ? int(P_COUNT) : int(kPlainPatterns); }
    const Stats& stats() const { return stats_; }
    void reset_stats() { stats_ = Stats(); }

    // A new operation. Returns the first non-zero status of what had to be enqueued.
    int push(const Rec& r, Sink& sink) {
        ++stats_.calls;
        int st = 0;
        if (pending_ >= 0 || count_ == kQueue) st = flush(sink);
        q_[count_++] = r;
        const int st2 = settle(sink);
        return st != 0 ? st : st2;
    }

    // Everything held is enqueued unfused, in call order.
    int flush(Sink& sink) {
        int st = 0;
        pending_ = -1;
        for (int i = 0; i < count_; ++i) {
            const int s = sink.primitive(q_[i]);
            ++stats_.unfused;
            if (st == 0) st = s;
        }
        count_ = 0;
        ncands_ = 0;
        judged_ = 0;
        return st;
    }

    // The pool got [p, p + bytes) back. Completes a pattern that waits for its temporaries.
    int note_free(const void* p, size_t bytes, Sink& sink) {
        if (pending_ < 0) return 0;
        const Pattern& P = patterns()[pending_];
        const char* lo = static_cast<const char*>(p);
        bool all = true;
        for (int t = 0; t < P.ntemps; ++t) {
            const Var& v = pending_match_.v[P.temps[t]];
            if (v.p >= lo && v.p + v.len <= lo + bytes) dead_ |= 1u << t;
            all = all && ((dead_ >> t) & 1u);
        }
        if (!all) return 0;
        const int st = emit_fused(P, pending_match_, sink);
        pending_ = -1;
        return st;
    }

    // An operation that is not held (a matrix product) reads rd[] and writes wr[]: true if it touches
    // nothing that a held operation writes and writes nothing that a held operation reads, so that it
    // may be enqueued ahead of them.
    bool independent(const char* const* rd, const size_t* rd_len, int nrd, const char* const* wr,
                     const size_t* wr_len, int nwr) const {
        for (int i = 0; i < count_; ++i) {
            const Rec& r = q_[i];
            for (int s = 0; s < r.nptr; ++s) {
                const bool written = (r.wr >> s) & 1;
                for (int k = 0; k < nwr; ++k)
                    if (ranges_overlap(r.p[s], r.len[s], wr[k], wr_len[k])) return false;
                if (written)
                    for (int k = 0; k < nrd; ++k)
                        if (ranges_overlap(r.p[s], r.len[s], rd[k], rd_len[k])) return false;
            }
        }
        return true;
    }
    void count_overtaken() { ++stats_.overtaken; }

private:
    // A pattern that agrees with the held calls so far (all of them, or its whole length).
    struct Candidate {
        int pattern;
        int matched;
        Match m;
    };

    int emit_fused(const Pattern& P, const Match& m, Sink& sink) {
        const int st = sink.fused(P, m, q_);
        ++stats_.fused;
        ++stats_.per_pattern[P.id];
        stats_.fused_calls += static_cast<uint64_t>(P.len);
        drop_front(P.len);
        return st;
    }

    void drop_front(int k) {
        if (k < count_) memmove(static_cast<void*>(q_), static_cast<const void*>(q_ + k), sizeof(Rec) * size_t(count_ - k));
        count_ -= k;
        ncands_ = 0;        // the candidates were anchored at the old first call
        judged_ = 0;
    }

    // Brings the candidates up to date with the held calls: from scratch when the first held call has
    // changed, else by looking at the calls that arrived since (one, as a rule).
    void update_candidates() {
        const Pattern* table = patterns();
        if (judged_ == 0) {
            ncands_ = 0;
            for (int k = 0; k < npatterns_; ++k) {
                const Pattern& P = table[k];
                if (P.e[0].kind != q_[0].kind) continue;      // most sequences open with another kind of call
                Candidate& c = cands_[ncands_];
                const int got = match_prefix(P, q_, count_, c.m);
                if (got < 0) continue;
                c.pattern = k;
                c.matched = got;
                ++ncands_;
            }
        } else {
            int kept = 0;
            for (int k = 0; k < ncands_; ++k) {
                Candidate& c = cands_[k];
                const Pattern& P = table[c.pattern];
                bool alive = true;
                while (alive && c.matched < count_ && c.matched < P.len) {
                    alive = match_call(P, c.matched, q_[c.matched], c.m);
                    if (alive) ++c.matched;
                }
                if (!alive) continue;
                if (kept != k) cands_[kept] = c;
                ++kept;
            }
            ncands_ = kept;
        }
        judged_ = count_;
    }

    int settle(Sink& sink) {
        int st = 0;
        const Pattern* table = patterns();
        while (count_ > 0) {
            update_candidates();
            bool partial = false, emitted = false;
            for (int k = 0; k < ncands_ && !emitted; ++k) {
                Candidate& c = cands_[k];
                const Pattern& P = table[c.pattern];
                if (c.matched < P.len) { partial = true; continue; }
                if (!fusable(P, c.m, q_)) { c.matched = -1; continue; }
                if (P.ntemps > 0) {
                    if (count_ != P.len) { c.matched = -1; continue; }     // calls follow: the temporaries are still alive
                    pending_ = c.pattern;
                    pending_match_ = c.m;
                    dead_ = 0;
                    return st;
                }
                const Match m = c.m;      // emit_fused drops the candidates
                const int s = emit_fused(P, m, sink);
                if (st == 0) st = s;
                emitted = true;
            }
            if (emitted) continue;
            if (partial) {
                // complete candidates that cannot be fused are done with
                int kept = 0;
                for (int k = 0; k < ncands_; ++k)
                    if (cands_[k].matched >= 0 && cands_[k].matched < table[cands_[k].pattern].len) {
                        if (kept != k) cands_[kept] = cands_[k];
                        ++kept;
                    }
                ncands_ = kept;
                return st;
            }
            const int s = sink.primitive(q_[0]);
            ++stats_.unfused;
            if (st == 0) st = s;
            drop_front(1);
        }
        return st;
    }

    Rec q_[kQueue];
    int count_ = 0;
    Candidate cands_[P_COUNT];
    int ncands_ = 0;
    int npatterns_ = kPlainPatterns;
    int judged_ = 0;           // held calls that the candidates have been compared with (0: candidates not built)
    int pending_ = -1;         // pattern that is complete and waits for its temporaries to be freed
    Match pending_match_;
    unsigned dead_ = 0;
    Stats stats_;
};

}  // namespace window
}  // namespace bship
