// matmul_mfma.hip -- MFMA GEMM for f32 / f16 / bf16 with f32 accumulation.
#include "common.hpp"

namespace aixk {

int matmul_mfma(aixk_ctx*, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*)
{
    return -1;      // not handled: caller uses the tiled kernel
}

} // namespace aixk
