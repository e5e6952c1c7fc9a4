// Instances of the i8 MFMA GEMM kernels: many-digit operands whose shift + 64 result bits end below 2^96 or 2^64: fewer digit pairs.
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_pruned(std::vector<Instance> &out)
{
    out.push_back(make_instance<9, 9, false, 12>());
    out.push_back(make_instance<9, 9, false, 8>());
    out.push_back(make_instance<9, 5, false, 8>());
    out.push_back(make_instance<5, 9, false, 8>());
}

}  // namespace zk
