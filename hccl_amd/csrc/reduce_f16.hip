// Fused reduce kernels for fp16 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::HalfSumOps<false>;
using Ops1 = detail::HalfProdOps;
using Ops2 = detail::HalfSelectOps<false, detail::kMax>;
using Ops3 = detail::HalfSelectOps<false, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT4(SelectReduceF16, Ops0, Ops1, Ops2, Ops3)

}  // namespace hccl_amd
