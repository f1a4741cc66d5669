// Fold kernels for element type uint32_t (see vrank_fold_impl.hpp).
#include "vrank_fold_impl.hpp"

namespace MegRay {
namespace vrank {
namespace detail {
MEGRAY_VRANK_INSTANTIATE(uint32_t)
}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
