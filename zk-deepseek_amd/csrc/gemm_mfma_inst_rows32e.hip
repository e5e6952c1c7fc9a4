// Instances of the i8 MFMA GEMM kernels: 32-row tiles, int32 weights only, two MFMA depths per step: (3,4) for
// activations of up to 23 bits against weights of up to 31 (an expert's first two products on a Q23 activation,
// inference/model.py:1271-1272, which would otherwise run on (4,4): a third more digit pairs).
#include "gemm_mfma_kernels.h"

namespace zk {

void mfma_instances_rows32e(std::vector<Instance> &out)
{
    out.push_back(make_instance<3, 4, true, 16, 2, true>());
}

}  // namespace zk
