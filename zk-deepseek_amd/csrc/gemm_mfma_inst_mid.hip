// Instances of the i8 MFMA GEMM kernels: (5,5) (6,5) (3,5) (6,3) (4,5).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_mid(std::vector<Instance> &out)
{
    out.push_back(make_instance<5, 5>());
    out.push_back(make_instance<6, 5>());
    out.push_back(make_instance<3, 5>());
    out.push_back(make_instance<6, 3>());
    out.push_back(make_instance<4, 5>());
}

}  // namespace zk
