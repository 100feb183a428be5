// BF16 storage: instantiates the forward and backward entry of libdsdpa.so for this type.
#include "dsdpa_impl.h"

namespace dsdpa {
template int fwd_impl<BF16>(const void *, const void *, const void *, const float *, void *, float *, void *, int, int, int, int,
                           int, int, int, float, const long long *, void *, bool);
template int bwd_impl<BF16>(const void *, const void *, const void *, const float *, const void *, const float *,
                           const void *, void *, void *, void *, float *, void *, int, int, int, int, int, int, int, float,
                           const long long *, unsigned, void *);
}  // namespace dsdpa
