// Instances of the i8 MFMA GEMM kernels: 32-row tiles for grouped launches on prepared three-digit planes of B, two depths
// per step (more bytes of planes in flight): (3,3) (4,3) (5,3).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_rows32c(std::vector<Instance> &out)
{
    out.push_back(make_instance<3, 3, true, 16, 2, false, true>());
    out.push_back(make_instance<4, 3, true, 16, 2, false, true>());
    out.push_back(make_instance<5, 3, true, 16, 2, false, true>());
}

}  // namespace zk
