// Small device-side helpers shared by the kernel files.
#ifndef LUTGEMM_DEVICE_UTIL_H
#define LUTGEMM_DEVICE_UTIL_H

#include <stdint.h>

#include <type_traits>
#include <utility>

namespace lutgemm_kernels {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// compile-time loop: body(std::integral_constant<int, I>) for I in [0, N)
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&body, std::integer_sequence<int, Is...>)
{
    (body(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&body)
{
    static_for_impl(body, std::make_integer_sequence<int, N>{});
}

}  // namespace lutgemm_kernels
#endif
