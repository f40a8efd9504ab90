// Bounds-checked buffer loads of 1-4 consecutive floats, for inner loops that must issue every load
// unconditionally (a load at a byte offset beyond the resource returns zeros without touching memory, so
// "no load" is an offset, not a branch, and the compiler can count outstanding loads exactly).
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

namespace bship {

constexpr int kBufferOob = 0x40000000;            // a byte offset beyond any resource made here (< 1 GiB)

template <int N> struct Piece { float v[N]; };    // N consecutive floats, aligned to 4 bytes only

// a buffer resource over `bytes` bytes at p; p and bytes are the same in every lane, and saying so keeps
// the descriptor in scalar registers
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_rsrc(const float* p, int bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(p);
    float* const q = reinterpret_cast<float*>(
        (static_cast<uint64_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(addr >> 32))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(addr))));
    return __builtin_amdgcn_make_buffer_rsrc(q, 0, __builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

template <int N>
__device__ __forceinline__ Piece<N> load_piece(__amdgpu_buffer_rsrc_t rsrc, int voff) {
    if constexpr (N == 1) return __builtin_bit_cast(Piece<1>, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, 0, 0));
    else if constexpr (N == 2) return __builtin_bit_cast(Piece<2>, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, 0, 0));
    else if constexpr (N == 3) {
        // four floats loaded, three kept (the 96-bit builtin does not load all three with this compiler;
        // written this way the compiler emits a 96-bit load itself)
        const Piece<4> q = __builtin_bit_cast(Piece<4>, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 0));
        Piece<3> p;
        p.v[0] = q.v[0]; p.v[1] = q.v[1]; p.v[2] = q.v[2];
        return p;
    }
    else return __builtin_bit_cast(Piece<4>, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 0));
}

}  // namespace bship
