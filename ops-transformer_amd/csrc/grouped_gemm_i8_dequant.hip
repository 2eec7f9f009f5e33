// Expert-grouped int8 GEMM: the kernels of the kDequant epilogue (see grouped_gemm_i8_kernels.h).
#include "grouped_gemm_i8_kernels.h"

namespace gemm {

hipError_t LaunchRingDequant(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchStreamShape<Epilogue::kDequant>(plan, args, sched, stream);
}

hipError_t LaunchGenericDequant(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchGenericShape<Epilogue::kDequant>(plan, args, sched, stream);
}

}  // namespace gemm
