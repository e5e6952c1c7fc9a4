// Instances of the i8 MFMA GEMM kernels: (3,3) (4,3) (4,4) (5,4).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_narrow(std::vector<Instance> &out)
{
    out.push_back(make_instance<3, 3>());
    out.push_back(make_instance<4, 3>());
    out.push_back(make_instance<4, 4>());
    out.push_back(make_instance<5, 4>());
}

}  // namespace zk
