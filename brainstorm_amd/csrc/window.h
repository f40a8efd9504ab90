// Library side of the fusing window (window_core.h): the queue behind the public entry points.
#pragma once

#include "common.h"
#include "window_core.h"

namespace bship {

// Hands an operation to the window. Returns the status of whatever had to be enqueued.
int window_push(const window::Rec& r);
// The pool got [p, p + bytes) back.
int window_note_free(const void* p, size_t bytes);
// A matrix product that reads rd[] and writes wr[] is about to be enqueued: held operations that
// it depends on (or that depend on it) are enqueued first; otherwise it overtakes them.
int window_before_product(const void* const* rd, const size_t* rd_len, int nrd, const void* const* wr,
                          const size_t* wr_len, int nwr);

// fused.hip: batch normalisation forward (training) with the scalars as the layer's calls carry them
int batchnorm_fwd_train_launch(const float* inputs, const float* gamma, const float* beta, float* mu, float* sigma,
                               float* sigma_b, float* centered, float* x_hat, float* out, int64_t M, int64_t N,
                               float neg_inv_m, float decay_mu, float rest_mu, float inv_m, float eps,
                               float decay_sigma, float rest_sigma);

}  // namespace bship
