// Instances of the i8 MFMA GEMM kernels: 32-row tiles: (3,3) (5,5), and (4,4) (4,5) for 28-bit activations against 31-bit weights (what an expert sees after the
// norm, inference/model.py:1017, 1324).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_rows32(std::vector<Instance> &out)
{
    out.push_back(make_instance<3, 3, true>());
    out.push_back(make_instance<5, 5, true>());
    out.push_back(make_instance<4, 4, true>());
    out.push_back(make_instance<4, 5, true>());
}

}  // namespace zk
