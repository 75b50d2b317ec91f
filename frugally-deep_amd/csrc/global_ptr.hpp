// Pointers typed with the global address space, for device code whose pointers do not come straight from kernel
// arguments.  A pointer read back from a structure in LDS is a generic one to the compiler: loads through it are flat
// instructions, which count against the LDS counter as well as the vector-memory one, so that every wait for an LDS read
// also waits for them.  Dereferencing through gptr<T> makes them global loads.
#pragma once

namespace fdx {

template <typename T>
using gptr = T __attribute__((address_space(1)))*;

template <typename T>
__device__ __forceinline__ gptr<T> as_global(T* q)
{
    return (gptr<T>)q;
}

} // namespace fdx
