// Instances of the 128 x 128 kernel for digit planes on both sides (gemm_mfma_pipe.h): three digits a side.
#include "gemm_mfma_kernels.h"
#include "gemm_mfma_pipe.h"

namespace zk {

MfmaKernel pipe_kernel(int na, int nb)
{
    if (na == 3 && nb == 3) return gemm_mfma_pipe_kernel<3, 3>;
    return nullptr;
}

size_t pipe_lds_size(int na, int nb) { return pipe_lds_bytes(na, nb); }

}  // namespace zk
