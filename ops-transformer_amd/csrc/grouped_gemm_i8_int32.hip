// Expert-grouped int8 GEMM: the kernels of the kInt32 epilogue (see grouped_gemm_i8_kernels.h).
#include "grouped_gemm_i8_kernels.h"

namespace gemm {

hipError_t LaunchRingInt32(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchStreamShape<Epilogue::kInt32>(plan, args, sched, stream);
}

hipError_t LaunchGenericInt32(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchGenericShape<Epilogue::kInt32>(plan, args, sched, stream);
}

}  // namespace gemm
