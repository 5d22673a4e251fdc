// The int8 GEMM instantiated for 4-byte outputs: int32 accumulators and binary32 (see gemm_i8_impl.hpp).
#include "gemm_i8_impl.hpp"

namespace i8f {
namespace gemm {
template int launch<OUT_I32>(GemmArgs &, hipStream_t);
template int launch<OUT_F32>(GemmArgs &, hipStream_t);
template int launch_group<OUT_F32>(GemmArgs *, int, hipStream_t);
}  // namespace gemm
}  // namespace i8f
