// Expert-grouped int8 GEMM: the kernels of the kSwiglu epilogue (see grouped_gemm_i8_kernels.h).
#include "grouped_gemm_i8_kernels.h"

namespace gemm {

hipError_t LaunchRingSwiglu(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchStreamShape<Epilogue::kSwiglu>(plan, args, sched, stream);
}

hipError_t LaunchGenericSwiglu(const Plan& plan, const KernelArgs& args, const int32_t* sched, hipStream_t stream) {
    return LaunchGenericShape<Epilogue::kSwiglu>(plan, args, sched, stream);
}

}  // namespace gemm
