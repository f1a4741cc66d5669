// Fold kernels for element type _Float16 (see vrank_fold_impl.hpp).
#include "vrank_fold_impl.hpp"

namespace MegRay {
namespace vrank {
namespace detail {
MEGRAY_VRANK_INSTANTIATE(_Float16)
}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
