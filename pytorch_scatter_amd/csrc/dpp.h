// Cross-lane moves with a fixed pattern, done in the vector ALU of gfx950 instead of through the LDS crossbar.
//
// __shfl / __shfl_up / __shfl_down / __shfl_xor compile to ds_bpermute_b32: an address computed per lane (two VALU
// instructions), an LDS instruction and a wait for its return. Where the pattern is known at compile time the same
// move is one v_mov_b32_dpp (often folded into the arithmetic instruction that uses it) or one v_permlane*_swap:
//   * inside a row of 16 lanes: quad_perm, row_shl / row_shr / row_ror, row_mirror (DPP);
//   * one lane across the whole wavefront: wave_shr:1 (DPP);
//   * rows to their neighbours: row_bcast:15 / row_bcast:31 (DPP, for scans), v_permlane16_swap and
//     v_permlane32_swap (new in gfx950) for an exchange of rows 0<->1, 2<->3 and of the two halves.
// Data-dependent lanes (a leader found by a ballot, a slot computed from a mask) keep __shfl.
// Like every cross-lane move these must be executed by the source lanes too: call them in a statement of their own,
// never inside one arm of a conditional that some source lanes do not take (a lane that reads a lane that is
// switched off gets its own value back).
//
// All helpers are for 4-byte values; lane_*64 wrap them for 8-byte values. "row" = 16 consecutive lanes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ts {

namespace dpp {
constexpr int kQuadXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kQuadXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kRowShl = 0x100;         // + n: lane i reads lane i + n of its row
constexpr int kRowShr = 0x110;         // + n: lane i reads lane i - n of its row
constexpr int kRowRor = 0x120;         // + n: rotate right inside the row
constexpr int kWaveShr1 = 0x138;       // lane i reads lane i - 1 of the wavefront
constexpr int kRowBcast15 = 0x142;     // lane 15 of every row to the whole next row
constexpr int kRowBcast31 = 0x143;     // lane 31 to rows 2 and 3

template <typename T> __device__ __forceinline__ int as_int(T x) {
  static_assert(sizeof(T) == 4, "4-byte values");
  int r;
  __builtin_memcpy(&r, &x, 4);
  return r;
}
template <typename T> __device__ __forceinline__ T from_int(int x) {
  T r;
  __builtin_memcpy(&r, &x, 4);
  return r;
}
// lanes without a source (or switched off by the masks) keep `old`
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, typename T>
__device__ __forceinline__ T mov(T old, T x) {
  return from_int<T>(__builtin_amdgcn_update_dpp(as_int(old), as_int(x), CTRL, ROW_MASK, BANK_MASK, false));
}
}  // namespace dpp

// value of lane i - 1; lane 0 keeps its own (what __shfl_up(x, 1) returns)
template <typename T> __device__ __forceinline__ T lane_up1(T x) {
#if defined(TS_DPP_OFF)  // build switch for measurements: every helper of this file through the LDS crossbar again
  return __shfl_up(x, 1);
#else
  return dpp::mov<dpp::kWaveShr1>(x, x);
#endif
}
__device__ __forceinline__ int64_t lane_up1_64(int64_t x) {
  const int lo = lane_up1((int)(uint32_t)x), hi = lane_up1((int)(x >> 32));
  return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
}

// value of lane i ^ OFF, OFF a power of two below 64 (what __shfl_xor(x, OFF) returns)
template <int OFF, typename T> __device__ __forceinline__ T lane_xor(T x) {
  static_assert(OFF == 1 || OFF == 2 || OFF == 4 || OFF == 8 || OFF == 16 || OFF == 32, "power of two below 64");
#if defined(TS_DPP_OFF)
  return __shfl_xor(x, OFF);
#endif
  if constexpr (OFF == 1) {
    return dpp::mov<dpp::kQuadXor1>(x, x);
  } else if constexpr (OFF == 2) {
    return dpp::mov<dpp::kQuadXor2>(x, x);
  } else if constexpr (OFF == 4) {
    // banks of four lanes: banks 0 and 2 read four lanes up, banks 1 and 3 four lanes down
    const T up = dpp::mov<dpp::kRowShl + 4, 0xf, 0x5>(x, x);
    return dpp::mov<dpp::kRowShr + 4, 0xf, 0xa>(up, x);
  } else if constexpr (OFF == 8) {
    return dpp::mov<dpp::kRowRor + 8>(x, x);
  } else if constexpr (OFF == 16) {
    // rows r0 r1 r2 r3 -> first result r0 r0 r2 r2, second r1 r1 r3 r3
    const auto s = __builtin_amdgcn_permlane16_swap((unsigned)dpp::as_int(x), (unsigned)dpp::as_int(x), false, false);
    return dpp::from_int<T>((int)(((threadIdx.x & 16) != 0) ? s[0] : s[1]));
  } else {
    // halves lo hi -> first result lo lo, second hi hi
    const auto s = __builtin_amdgcn_permlane32_swap((unsigned)dpp::as_int(x), (unsigned)dpp::as_int(x), false, false);
    return dpp::from_int<T>((int)(((threadIdx.x & 32) != 0) ? s[0] : s[1]));
  }
}

// value of lane i + OFF for the lanes whose bit OFF is clear (the receiving side of a reduction tree in which lane
// i takes lane i + OFF: OFF = 32, 16, ... down to 1, the result in lane 0 of the group); the other lanes receive
// an unspecified lane's value, which such a tree never uses
template <int OFF, typename T> __device__ __forceinline__ T lane_down(T x) {
  static_assert(OFF == 1 || OFF == 2 || OFF == 4 || OFF == 8 || OFF == 16 || OFF == 32, "power of two below 64");
#if defined(TS_DPP_OFF)
  return __shfl_down(x, OFF);
#endif
  if constexpr (OFF < 16) {
    return dpp::mov<dpp::kRowShl + OFF>(x, x);
  } else if constexpr (OFF == 16) {
    const auto s = __builtin_amdgcn_permlane16_swap((unsigned)dpp::as_int(x), (unsigned)dpp::as_int(x), false, false);
    return dpp::from_int<T>((int)s[1]);
  } else {
    const auto s = __builtin_amdgcn_permlane32_swap((unsigned)dpp::as_int(x), (unsigned)dpp::as_int(x), false, false);
    return dpp::from_int<T>((int)s[1]);
  }
}

// the same moves for values of any size up to 8 bytes (smaller ones travel in a 32-bit register, 8-byte ones as
// two halves)
template <int OFF, bool XOR, typename T> __device__ __forceinline__ T lane_move_any(T x) {
  static_assert(sizeof(T) <= 8, "at most 8 bytes");
  if constexpr (sizeof(T) == 4) {
    return XOR ? lane_xor<OFF>(x) : lane_down<OFF>(x);
  } else if constexpr (sizeof(T) < 4) {
    int w = 0;
    __builtin_memcpy(&w, &x, sizeof(T));
    w = XOR ? lane_xor<OFF>(w) : lane_down<OFF>(w);
    T r;
    __builtin_memcpy(&r, &w, sizeof(T));
    return r;
  } else {
    int w[2];
    __builtin_memcpy(w, &x, 8);
    w[0] = XOR ? lane_xor<OFF>(w[0]) : lane_down<OFF>(w[0]);
    w[1] = XOR ? lane_xor<OFF>(w[1]) : lane_down<OFF>(w[1]);
    T r;
    __builtin_memcpy(&r, w, 8);
    return r;
  }
}
template <int OFF, typename T> __device__ __forceinline__ T lane_xor_any(T x) { return lane_move_any<OFF, true>(x); }
template <int OFF, typename T> __device__ __forceinline__ T lane_down_any(T x) { return lane_move_any<OFF, false>(x); }

// Butterfly among the `lanes` neighbouring lanes of a group (a power of two up to 64, the same for the whole
// wavefront): x = op(x, value of lane ^ off) for off = lanes / 2 down to 1, as a loop over __shfl_xor would do it
// (same partners, same order, so also the same bits for floating-point sums); every lane ends with the result.
template <typename T, typename Op> __device__ __forceinline__ T group_butterfly(T x, int lanes, Op op) {
  if (lanes > 32) x = op(x, lane_xor_any<32>(x));
  if (lanes > 16) x = op(x, lane_xor_any<16>(x));
  if (lanes > 8) x = op(x, lane_xor_any<8>(x));
  if (lanes > 4) x = op(x, lane_xor_any<4>(x));
  if (lanes > 2) x = op(x, lane_xor_any<2>(x));
  if (lanes > 1) x = op(x, lane_xor_any<1>(x));
  return x;
}

// inclusive prefix sum over the 64 lanes of a wavefront (int32): four steps inside the rows, then lane 15 of rows 0
// and 2 into rows 1 and 3, then lane 31 into rows 2 and 3
__device__ __forceinline__ int wave_inclusive_sum(int x) {
#if defined(TS_DPP_OFF)
  const int lane = threadIdx.x & 63;
  for (int d = 1; d < 64; d <<= 1) {
    const int y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  return x;
#endif
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowShr + 1, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowShr + 2, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowShr + 4, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowShr + 8, 0xf, 0xf, true);
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowBcast15, 0xa, 0xf, false);
  x += __builtin_amdgcn_update_dpp(0, x, dpp::kRowBcast31, 0xc, 0xf, false);
  return x;
}

}  // namespace ts
