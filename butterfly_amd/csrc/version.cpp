// torch_butterfly::cuda_version for the package initialiser.
//
// The reference registers this operator from csrc/version.cpp:14-23 and returns
// CUDA_VERSION, or -1 for a build without CUDA.  This library is HIP only, so the answer
// is always -1; the HIP runtime version is exposed as torch_butterfly::hip_version by the
// operator library.

#include <torch/library.h>

namespace {
int64_t cuda_version() { return -1; }
}  // namespace

TORCH_LIBRARY_FRAGMENT(torch_butterfly, m) { m.def("cuda_version", cuda_version); }
