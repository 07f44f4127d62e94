// Which backend this build of the `deep_ep._C` extension drives.  Exactly one platform macro is defined by the
// build (the role of csrc/platform/config.hpp:5-17 in the reference, which knows "cuda" and "ascend").
#pragma once

#include <string_view>

#if !defined(DEEP_EP_PLATFORM_HIP)
#error "Define exactly one DeepEP platform macro (this tree builds with -DDEEP_EP_PLATFORM_HIP)"
#endif
#if defined(DEEP_EP_PLATFORM_CUDA) || defined(DEEP_EP_PLATFORM_ASCEND)
#error "Define exactly one DeepEP platform macro"
#endif

namespace deep_ep::platform {

inline constexpr std::string_view kName = "hip";

}  // namespace deep_ep::platform
