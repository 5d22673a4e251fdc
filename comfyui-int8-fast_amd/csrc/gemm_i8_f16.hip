// The int8 GEMM instantiated for binary16 outputs (see gemm_i8_impl.hpp).
#include "gemm_i8_impl.hpp"

namespace i8f {
namespace gemm {
template int launch<OUT_F16>(GemmArgs &, hipStream_t);
template int launch_group<OUT_F16>(GemmArgs *, int, hipStream_t);
}  // namespace gemm
}  // namespace i8f
