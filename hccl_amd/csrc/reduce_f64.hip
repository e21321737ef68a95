// Fused reduce kernels for fp64 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::FpOps<double, detail::kSum>;
using Ops1 = detail::FpOps<double, detail::kProd>;
using Ops2 = detail::FpOps<double, detail::kMax>;
using Ops3 = detail::FpOps<double, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT4(SelectReduceF64, Ops0, Ops1, Ops2, Ops3)

}  // namespace hccl_amd
