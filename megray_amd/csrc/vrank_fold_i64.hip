// Fold kernels for element type int64_t (see vrank_fold_impl.hpp).
#include "vrank_fold_impl.hpp"

namespace MegRay {
namespace vrank {
namespace detail {
MEGRAY_VRANK_INSTANTIATE(int64_t)
}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
