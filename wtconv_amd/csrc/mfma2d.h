// Internal interface of the matrix-core (MFMA) 2-D path; implemented in mfma2d.hip.
#pragma once

#include <stddef.h>

#include "common.h"
#include "wgrad_finish.h"

namespace wt {

// Whether a forward / input-gradient pass of this shape runs on the MFMA kernels, and the
// workspace it then needs (none: the kernel folds the parameters of a channel itself).
struct Mfma2dQuery {
  bool ok;
  size_t ws_bytes;
};
Mfma2dQuery mfma2d_query(int B, int C, int H, int W, int K, int L, int dtype);

// One pass (flip = 0: forward, 1: input gradient).  Returns 0 or a WTCONV_E_* code with the
// message left in the thread's error buffer.  The kernel also clears the `nzero` words at `zero_words` (may be null).
int mfma2d_pass(const char* fn, const void* x, void* out, const wtconv_params* params, int B, int C, int H, int W,
                int K, int L, int dtype, int pdtype, hipStream_t stream, int flip, unsigned* zero_words = nullptr,
                int nzero = 0);

// Parameter gradients of bf16 tensors: whether the shape runs on the MFMA kernel, and the size of the
// per-chunk partial sums it leaves in the workspace (`nchunk` records per channel).
struct Mfma2dWgradQuery {
  bool ok;
  int nchunk;
  size_t ws_bytes;
};
Mfma2dWgradQuery mfma2d_wgrad_query(int B, int C, int H, int W, int K, int L, int dtype);

// `fin`: with tickets set, the kernel finishes the channels itself (no wgrad_finish_kernel launch after it).
int mfma2d_wgrad_pass(const char* fn, const void* x, const void* grad_out, float* partial, int B, int C, int H, int W,
                      int K, int L, const FinishArgs& fin, hipStream_t stream);

}  // namespace wt
