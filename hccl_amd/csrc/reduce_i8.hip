// Fused reduce kernels for int8 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::Int8Ops<detail::kSum>;
using Ops1 = detail::Int8Ops<detail::kProd>;
using Ops2 = detail::Int8Ops<detail::kMax>;
using Ops3 = detail::Int8Ops<detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT4(SelectReduceI8, Ops0, Ops1, Ops2, Ops3)

}  // namespace hccl_amd
