// Instances of the i8 MFMA GEMM kernels: the many-digit combinations (9,5) (5,9) (9,9).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_wide(std::vector<Instance> &out)
{
    out.push_back(make_instance<9, 5>());
    out.push_back(make_instance<5, 9>());
    out.push_back(make_instance<9, 9>());
}

}  // namespace zk
