// Fused reduce kernels for int32 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::IntOps<int32_t, uint32_t, detail::kSum>;
using Ops1 = detail::IntOps<int32_t, uint32_t, detail::kProd>;
using Ops2 = detail::IntOps<int32_t, uint32_t, detail::kMax>;
using Ops3 = detail::IntOps<int32_t, uint32_t, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT4(SelectReduceI32, Ops0, Ops1, Ops2, Ops3)

}  // namespace hccl_amd
