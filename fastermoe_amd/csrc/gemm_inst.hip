// One translation unit per (element type, product) of the grouped GEMM; the build
// compiles this file nine times with -DFMOE_GEMM_TYPE=<0 f32|1 bf16|2 f16> and
// -DFMOE_GEMM_PRODUCT=<0 fwd|1 dgrad|2 wgrad>.
#include "gemm_kernel.hpp"

#if FMOE_GEMM_TYPE == 0
#define FMOE_T float
#define FMOE_TNAME f32
#elif FMOE_GEMM_TYPE == 1
#define FMOE_T __bf16
#define FMOE_TNAME bf16
#elif FMOE_GEMM_TYPE == 2
#define FMOE_T _Float16
#define FMOE_TNAME f16
#else
#error "FMOE_GEMM_TYPE must be 0, 1 or 2"
#endif

#define FMOE_CAT_(a, b, c) launch_mfma_##a##_##b
#define FMOE_CAT(a, b) FMOE_CAT_(a, b, )

namespace fmoe {
using namespace gemm;

#if FMOE_GEMM_PRODUCT == 0
int FMOE_CAT(FMOE_TNAME, fwd)(GemmParams &prm, int epilogue, hipStream_t stream) {
    return launch_by_epilogue<FMOE_T, kKC, kKC, kRaggedRows, (1 << kEpiStore) | (1 << kEpiBiasAct)>(prm, epilogue, stream);
}
#elif FMOE_GEMM_PRODUCT == 1
int FMOE_CAT(FMOE_TNAME, dgrad)(GemmParams &prm, int epilogue, hipStream_t stream) {
    return launch_by_epilogue<FMOE_T, kMC, kKC, kRaggedRows, (1 << kEpiStore) | (1 << kEpiDAct)>(prm, epilogue, stream);
}
#elif FMOE_GEMM_PRODUCT == 2
int FMOE_CAT(FMOE_TNAME, wgrad)(GemmParams &prm, int epilogue, hipStream_t stream) {
    return launch_by_epilogue<FMOE_T, kMC, kMC, kRaggedK, (1 << kEpiStore)>(prm, epilogue, stream);
}
#else
#error "FMOE_GEMM_PRODUCT must be 0, 1 or 2"
#endif

}  // namespace fmoe
