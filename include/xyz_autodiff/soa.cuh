#pragma once
// 16-byte access to structure-of-arrays buffers.
//
// A kernel that evaluates one small graph per problem reads a handful of
// scalars and writes a handful of scalars per problem.  Laid out as one array
// per scalar (SoA), consecutive lanes touch consecutive addresses; letting
// each lane own four consecutive problems turns every access into one
// global_load_dwordx4 / global_store_dwordx4, 1 KiB per wavefront instruction,
// which is the widest transaction the memory pipeline offers.
//
// Quad<T> is the register image of four consecutive elements.  The *_stream
// variants mark the access non-temporal: data that is touched exactly once
// should not displace anything in L2.
//
// Not present in xyz-autodiff-cuda, whose examples keep parameters as arrays
// of 36-byte structs (examples/mini-gaussian-splatting/gaussian_parameters.h:12-18).

#include <cstddef>

#include <xyz_autodiff/detail/config.cuh>

namespace xyz_autodiff {
namespace soa {

template <typename T>
struct alignas(4 * sizeof(T)) Quad {
    T v[4];
    XAD_INLINE T& operator[](std::size_t i) { return v[i]; }
    XAD_INLINE const T& operator[](std::size_t i) const { return v[i]; }
};

// `base + 4 * group` must be aligned to 4 * sizeof(T) bytes.
template <typename T>
XAD_INLINE Quad<T> load4(const T* base, std::size_t group) {
    return *reinterpret_cast<const Quad<T>*>(base + 4 * group);
}

template <typename T>
XAD_INLINE void store4(T* base, std::size_t group, const Quad<T>& q) {
    *reinterpret_cast<Quad<T>*>(base + 4 * group) = q;
}

#if XAD_DEVICE_PASS
namespace detail {
template <typename T>
using native_quad = T __attribute__((ext_vector_type(4)));
}

template <typename T>
XAD_INLINE Quad<T> load4_stream(const T* base, std::size_t group) {
    using V = detail::native_quad<T>;
    const V raw = __builtin_nontemporal_load(reinterpret_cast<const V*>(base + 4 * group));
    return Quad<T>{{raw.x, raw.y, raw.z, raw.w}};
}

template <typename T>
XAD_INLINE void store4_stream(T* base, std::size_t group, const Quad<T>& q) {
    using V = detail::native_quad<T>;
    V raw = {q.v[0], q.v[1], q.v[2], q.v[3]};
    __builtin_nontemporal_store(raw, reinterpret_cast<V*>(base + 4 * group));
}
#else
template <typename T>
XAD_INLINE Quad<T> load4_stream(const T* base, std::size_t group) {
    return load4(base, group);
}
template <typename T>
XAD_INLINE void store4_stream(T* base, std::size_t group, const Quad<T>& q) {
    store4(base, group, q);
}
#endif

}  // namespace soa
}  // namespace xyz_autodiff
