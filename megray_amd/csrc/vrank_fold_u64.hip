// Fold kernels for element type uint64_t (see vrank_fold_impl.hpp).
#include "vrank_fold_impl.hpp"

namespace MegRay {
namespace vrank {
namespace detail {
MEGRAY_VRANK_INSTANTIATE(uint64_t)
}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
