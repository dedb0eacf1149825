// The HIP build of paperkiln's device seam: what a maintainer adds to the reference tree to run its tape on
// an MI355X through libpaperkiln_amd.so. Compile microtorch_hip_seam.cpp INTO the reference in place of
// src/device.cpp, src/device_cache.cpp, src/cuda_ops.cu and src/cuda_resident.cu; it defines every function
// include/microtorch/device.hpp:19-32 and include/microtorch/device_cache.hpp:19-127 declare, with the
// reference's own conventions (host Matrix in, host Matrix out, `false` = not handled, std::runtime_error on
// failure), and adds the entries below in the same style.
#pragma once
#include <cstddef>
#include <vector>

#include "microtorch/autograd.hpp"
#include "microtorch/device_cache.hpp"

namespace microtorch {
namespace device {
namespace devops {

// Forward of ops::fused_attention (src/ops.cpp:863-902) or, with window >= 1, of ops::swa_attention
// (src/ops.cpp:948-995) for one head: q, k, v are [rows, dk] with rows = B stacked sequences of seq_len
// (0 = one sequence). Writes y [rows, dk] and lse[rows], the per-row logsumexp of the scaled scores over the
// visible set -- all the backward needs besides q, k, v and y; no [T, T] matrix exists on either side.
bool attention_fwd(const Matrix& q, const Matrix& k, const Matrix& v, float scale, size_t seq_len, bool causal,
                   size_t window, size_t sinks, Matrix& y, std::vector<float>& lse);
// The closure of the same node (src/ops.cpp:902-933, 997-1026), recomputed from q, k and lse. A null
// output pointer means "not wanted"; the others must be sized [rows, dk] and are overwritten.
bool attention_bwd(const Matrix& q, const Matrix& k, const Matrix& v, const Matrix& y, const std::vector<float>& lse,
                   const Matrix& dy, float scale, size_t seq_len, bool causal, size_t window, size_t sinks, Matrix* dq,
                   Matrix* dk, Matrix* dv);
// ops::silu and its closure (src/ops.cpp:404-424).
bool silu_fwd(const Matrix& x, Matrix& y);
bool silu_bwd(const Matrix& x, const Matrix& dy, Matrix& dx);

}  // namespace devops
}  // namespace device

namespace ops {

// ops::fused_attention / ops::swa_attention as they read once the seam above is wired in: the same
// signatures (include/microtorch/ops.hpp:141-150), the device entry tried first and the host loops of
// src/ops.cpp kept as the "not handled" path, and a tape node that keeps y and lse instead of the [T, T]
// weight matrix the host closure captures (src/ops.cpp:876,902).
Var fused_attention_hip(const Var& q, const Var& k, const Var& v, float scale, size_t seq_len, bool causal);
Var swa_attention_hip(const Var& q, const Var& k, const Var& v, float scale, size_t window, size_t sinks,
                      size_t seq_len = 0);

}  // namespace ops
}  // namespace microtorch
