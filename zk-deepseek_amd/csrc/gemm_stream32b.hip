// Instances of the streamed 32-row grouped kernel (int32 weights), wider digit counts.
#include "gemm_stream32.h"

namespace zk {

MfmaKernel stream32_grouped_kernel_wide(int na, int nb, size_t *lds)
{
    MfmaKernel fn = nullptr;
#define ZK_S32(NA_, NB_) if (na == NA_ && nb == NB_) fn = gemm_stream32_grouped_kernel<NA_, NB_>
    ZK_S32(4, 5);
    ZK_S32(5, 3);
    ZK_S32(5, 4);
    ZK_S32(5, 5);
#undef ZK_S32
    if (fn && lds) *lds = stream32_lds_bytes(na);
    return fn;
}

}  // namespace zk
