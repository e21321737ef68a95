// Fused reduce kernels for bf16 (all reduce ops this type admits).
#include "reduce_kernel_impl.h"

namespace hccl_amd {
namespace {
using Ops0 = detail::HalfSumOps<true>;
using Ops1 = detail::HalfSelectOps<true, detail::kMax>;
using Ops2 = detail::HalfSelectOps<true, detail::kMin>;
}  // namespace

HCCL_AMD_DEFINE_SELECT3(SelectReduceBf16, Ops0, Ops1, Ops2)

}  // namespace hccl_amd
