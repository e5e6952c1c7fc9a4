// Instances of the i8 MFMA GEMM kernels: 32-row tiles for grouped launches on prepared four-digit planes of B (int32
// weights), two depths per step: (4,4) (5,4).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_rows32d(std::vector<Instance> &out)
{
    out.push_back(make_instance<4, 4, true, 16, 2, false, true>());
    out.push_back(make_instance<5, 4, true, 16, 2, false, true>());
}

}  // namespace zk
