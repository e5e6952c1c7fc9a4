// Instances of the i8 MFMA GEMM kernels: 32-row tiles: the int32-only forms of (3,3) and (4,4) with two depths per step, and
// (4,3) (5,3) for wider activations against prepared three-digit weight planes (whose digit count a kernel has to match
// exactly).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_rows32b(std::vector<Instance> &out)
{
    out.push_back(make_instance<3, 3, true, 16, 2, true>());
    out.push_back(make_instance<4, 4, true, 16, 2, true>());
    out.push_back(make_instance<4, 3, true>());
    out.push_back(make_instance<5, 3, true>());
}

}  // namespace zk
