// Fused reduce kernels for fp32 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::FpOps<float, detail::kSum>;
using Ops1 = detail::FpOps<float, detail::kProd>;
using Ops2 = detail::FpOps<float, detail::kMax>;
using Ops3 = detail::FpOps<float, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT4(SelectReduceF32, Ops0, Ops1, Ops2, Ops3)

}  // namespace hccl_amd
