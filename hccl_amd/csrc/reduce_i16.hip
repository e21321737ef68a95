// Fused reduce kernels for int16 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::IntOps<int16_t, uint16_t, detail::kSum>;
using Ops1 = detail::IntOps<int16_t, uint16_t, detail::kMax>;
using Ops2 = detail::IntOps<int16_t, uint16_t, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT3(SelectReduceI16, Ops0, Ops1, Ops2)

}  // namespace hccl_amd
