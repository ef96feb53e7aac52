// One instantiation of the 256x256 GEMM kernel per translation unit (the kernel's
// K step is a single unrolled body of 128 MFMAs and takes minutes to compile):
// built six times with -DFO_INST_DTYPE={0,1} (fp16, bf16) and -DFO_INST_MODE={0,1,2}
// (plain, signal, scatter epilogue).
#include "fo_gemm256_kernel.h"
#include "fo_gemm_launch.h"

#if !defined(FO_INST_DTYPE) || !defined(FO_INST_MODE)
#error "compile with -DFO_INST_DTYPE=0|1 -DFO_INST_MODE=0|1|2"
#endif

namespace fo_gemm_dev {

#define FO_CAT3_(a, b, c, d) a##b##c##d
#define FO_CAT3(a, b, c, d) FO_CAT3_(a, b, c, d)

#if FO_INST_DTYPE == 0
typedef fo_f16_tag inst_tag;
#else
typedef fo_bf16_tag inst_tag;
#endif

int FO_CAT3(fo_gemm256_launch_, FO_INST_DTYPE, _, FO_INST_MODE)(const GemmArgs &a, hipStream_t stream, int *resident_out,
                                                             int expect_resident) {
    return launch_kernel<fo_gemm256_kernel<inst_tag, FO_INST_MODE>, kSmem256, 256>(a, stream, resident_out, expect_resident);
}

}  // namespace fo_gemm_dev
