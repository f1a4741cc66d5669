// Fold kernels for element type double (see vrank_fold_impl.hpp).
#include "vrank_fold_impl.hpp"

namespace MegRay {
namespace vrank {
namespace detail {
MEGRAY_VRANK_INSTANTIATE(double)
}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
