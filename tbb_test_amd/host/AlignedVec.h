// aligned_vector<T>: std::vector whose storage starts on a 64-byte boundary, the host-side
// container the reference benchmark uses for flat buffers (reference AlignedVec.h:122-123).
// Written against the C++17 minimal-allocator requirements; allocator_traits supplies the rest.
#pragma once

#include <cstddef>
#include <cstdlib>
#include <limits>
#include <new>
#include <vector>

template <typename T, std::size_t Alignment>
struct aligned_allocator {
  static_assert((Alignment & (Alignment - 1)) == 0, "alignment must be a power of two");
  using value_type = T;

  template <typename U>
  struct rebind {
    using other = aligned_allocator<U, Alignment>;
  };

  aligned_allocator() noexcept = default;
  template <typename U>
  aligned_allocator(const aligned_allocator<U, Alignment>&) noexcept {}

  T* allocate(std::size_t n) {
    if (n == 0) return nullptr;
    if (n > std::numeric_limits<std::size_t>::max() / sizeof(T)) throw std::bad_array_new_length();
    // aligned_alloc wants a size that is a multiple of the alignment
    std::size_t bytes = (n * sizeof(T) + Alignment - 1) / Alignment * Alignment;
    void* p = std::aligned_alloc(Alignment, bytes);
    if (!p) throw std::bad_alloc();
    return static_cast<T*>(p);
  }

  void deallocate(T* p, std::size_t) noexcept { std::free(p); }

  template <typename U>
  bool operator==(const aligned_allocator<U, Alignment>&) const noexcept { return true; }
  template <typename U>
  bool operator!=(const aligned_allocator<U, Alignment>&) const noexcept { return false; }
};

template <typename T>
using aligned_vector = std::vector<T, aligned_allocator<T, 64>>;
