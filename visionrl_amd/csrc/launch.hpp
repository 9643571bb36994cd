// Kernel launches whose status is the launch's own return value: the thread's sticky "last error" is neither
// read (it may hold what an earlier, unrelated call left behind) nor cleared (that call's owner may still
// want it).
#pragma once

#include <hip/hip_runtime.h>

#include <tuple>
#include <utility>

namespace {

template <typename... P, typename... A>
int vrl_launch(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t stream, A &&...args) {
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    std::tuple<std::decay_t<P>...> values{static_cast<std::decay_t<P>>(std::forward<A>(args))...};   // as the kernel takes them
    return std::apply(
        [&](auto &...v) {
            void *slots[] = {static_cast<void *>(&v)...};
            return (int)hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, slots, lds, stream);
        },
        values);
}

}  // namespace
