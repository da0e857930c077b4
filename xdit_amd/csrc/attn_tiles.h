// Pieces shared by the 16-bit attention kernels: MFMA wrappers, the LDS tile geometry and the
// direct global->LDS load.
#pragma once
#include <utility>

#include "common.h"

namespace xdit {

constexpr int kKeysPerTile = 64;
// A row maximum is replaced only when it grows by more than this many powers of two, so the
// rescale of the output accumulator is skipped on almost every tile; exponentials stay <= 2^8.
constexpr float kLazyRescaleLog2 = 8.0f;

template <typename T> struct Mfma16;
template <> struct Mfma16<__bf16> {
  typedef bf16x8 vec8;
  typedef bf16x2 vec2;
  static __device__ __forceinline__ f32x16 mma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<_Float16> {
  typedef f16x8 vec8;
  typedef f16x2 vec2;
  static __device__ __forceinline__ f32x16 mma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// LDS layout of a K (or V) tile: 64 rows of D 16-bit elements.  K is read with ds_read_b128
// (lane -> one key row, 16 bytes), V with ds_read_b64_tr_b16 (16-lane group -> 4 key rows x 32
// bytes).  A direct global->LDS load writes lane i at LDS offset base + 16*i, i.e. one 1 KiB
// contiguous piece per wavefront instruction, so padding can only go BETWEEN those pieces.  Each
// piece therefore holds rows {g, g+NG, g+2NG, ...} (NG pieces per tile) and pieces are
// 1024 + PAD bytes apart: rows that are read together (consecutive rows) then sit in different
// pieces, PAD bytes apart in bank space (PAD = 16 for the 16-byte K reads, 64 for the 64-byte V
// reads), which makes both read patterns bank-conflict free while every read address is one
// per-lane base plus a compile-time immediate.
template <int D> struct TileGeom {
  static constexpr int ROW_BYTES = D * 2;
  static constexpr int ROWS_PER_PIECE = 1024 / ROW_BYTES;
  static constexpr int NG = kKeysPerTile / ROWS_PER_PIECE;
  static constexpr int K_PITCH = 1024 + 16;
  static constexpr int V_PITCH = 1024 + 64;
  static constexpr int K_BYTES = NG * K_PITCH;
  static constexpr int V_BYTES = NG * V_PITCH;
  static constexpr int BUF_BYTES = K_BYTES + V_BYTES;
};

// Direct global->LDS load of 16 bytes per lane: lane i's data lands at LDS address lds + 16*i.
// `base` (64-bit) and `lds` must be wavefront-uniform; `off` is the lane's byte offset from base.
// Issued as inline assembly so that the compiler does not order later LDS reads of OTHER tile
// buffers behind it; completion is awaited explicitly with s_waitcnt vmcnt(N).
__device__ __forceinline__ void load_lds_16(const void* base, unsigned off, unsigned lds) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(off), "s"(base)
      : "memory", "m0");
}

// Compile-time loop: f(std::integral_constant<int, I>) for I = 0..N-1.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}
// LDS reads issued by hand so that several are in flight.  The compiler does not know that the
// destination is still in flight, so before its first use it must go through lds_wait<N>(x) (or
// lds_wait2 for two registers): N is the number of LDS reads issued AFTER the one being awaited;
// LDS returns data in order, so "at most N outstanding" means that read has landed.  Reads the
// compiler issues in between only make the wait stricter.
template <int OFF, typename V>
__device__ __forceinline__ void lds_read_b128(V& dst, unsigned addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF, typename V>
__device__ __forceinline__ void lds_read_tr16_b64(V& dst, unsigned addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF, typename V>
__device__ __forceinline__ void lds_read_tr8_b64(V& dst, unsigned addr) {
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int N, typename V>
__device__ __forceinline__ void lds_wait(V& x) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N));
}
template <int N, typename V>
__device__ __forceinline__ void lds_wait2(V& x, V& y) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
}

template <int N, typename V>
__device__ __forceinline__ void lds_wait4(V& x, V& y, V& z, V& w) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(x), "+v"(y), "+v"(z), "+v"(w) : "n"(N));
}

}  // namespace xdit
