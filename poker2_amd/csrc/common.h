// Shared device helpers for the gfx950 kernels: combo tables, wave64 / block
// reductions and scans, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define P2_H 1326          // hole-card combos
#define P2_HPAIRS 663      // float2 pairs per 1326-float row (5304 B, 8-byte aligned)
#define P2_CARDS 52
#define P2_WAVE 64

// Every entry point returns hipError_t as int; argument errors use this value.
#define P2_EINVAL 1  // == hipErrorInvalidValue

#define P2_LAUNCH_CHECK()                         \
  do {                                            \
    hipError_t e__ = hipGetLastError();           \
    if (e__ != hipSuccess) return (int)e__;       \
  } while (0)

// combo index h -> its two cards (a < b), lexicographic order:
// h = a*(103-a)/2 + (b-a-1)   (src/p2/env/card_utils.py:58-68)
struct P2ComboTable {
  uint8_t a[P2_H];
  uint8_t b[P2_H];
  uint16_t row_start[P2_CARDS + 1];  // first index of combos whose low card is a
  constexpr P2ComboTable() : a(), b(), row_start() {
    int k = 0;
    for (int c1 = 0; c1 < P2_CARDS; ++c1) {
      row_start[c1] = (uint16_t)k;
      for (int c2 = c1 + 1; c2 < P2_CARDS; ++c2) {
        a[k] = (uint8_t)c1;
        b[k] = (uint8_t)c2;
        ++k;
      }
    }
    row_start[P2_CARDS] = (uint16_t)k;
  }
};

__device__ const P2ComboTable p2_combo = P2ComboTable();

__device__ __forceinline__ int p2_combo_index(int lo, int hi) {
  return (lo * (103 - lo)) / 2 + (hi - lo - 1);
}

// ---- wave64 primitives ------------------------------------------------------
// DPP move with zero fill: lanes without a source (row edge) read 0.
template <int CTRL>
__device__ __forceinline__ float p2_dpp0(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

// The two row-broadcast steps that end a wave scan: the last lane of row 0 / 2 is added to rows 1 / 3,
// then lane 31 to rows 2 and 3.  Written as the add with a DPP operand and a row mask (lanes of the
// masked rows keep their value); from the builtin the compiler makes a zero, a DPP move and an add for
// each.  The leading s_nop covers the wait states a DPP read needs after a VALU write of its source
// (2) or of EXEC (5), which nobody inserts around inline assembly; inside, the other value's
// instruction and one s_nop separate each write from the DPP read of the same register.
__device__ __forceinline__ void p2_scan_row_carries(float& a, float& b) {
  asm volatile(
      "s_nop 4\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void p2_scan_row_carries(float& a, float& b, float& c, float& d) {
  asm volatile(
      "s_nop 4\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_add_f32_dpp %2, %2, %2 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, %3, %3 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_add_f32_dpp %2, %2, %2 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_add_f32_dpp %3, %3, %3 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ void p2_scan_row_carries(float& a) {
  asm volatile(
      "s_nop 4\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(a));
}

// Inclusive prefix sum over the 64 lanes: four row shifts inside each 16-lane row, then two
// row broadcasts carry the row totals across (six VALU ops, no LDS traffic).
__device__ __forceinline__ float p2_wave_scan_incl(float v) {
  v += p2_dpp0<0x111>(v);  // row_shr:1
  v += p2_dpp0<0x112>(v);  // row_shr:2
  v += p2_dpp0<0x114>(v);  // row_shr:4
  v += p2_dpp0<0x118>(v);  // row_shr:8
  p2_scan_row_carries(v);
  return v;
}
__device__ __forceinline__ float p2_wave_scan_incl(float v, int /*lane*/) { return p2_wave_scan_incl(v); }

// Two independent scans in lockstep: each DPP step of one fills the two wait states the other
// needs between writing a register and reading it through DPP.
__device__ __forceinline__ void p2_wave_scan_incl2(float& a, float& b) {
  a += p2_dpp0<0x111>(a); b += p2_dpp0<0x111>(b);
  a += p2_dpp0<0x112>(a); b += p2_dpp0<0x112>(b);
  a += p2_dpp0<0x114>(a); b += p2_dpp0<0x114>(b);
  a += p2_dpp0<0x118>(a); b += p2_dpp0<0x118>(b);
  p2_scan_row_carries(a, b);
}

// Four scans in lockstep (two cards' lists of both players): every DPP step has three independent
// instructions between a register's write and its next DPP read.
__device__ __forceinline__ void p2_wave_scan_incl4(float& a, float& b, float& c, float& d) {
  a += p2_dpp0<0x111>(a); b += p2_dpp0<0x111>(b); c += p2_dpp0<0x111>(c); d += p2_dpp0<0x111>(d);
  a += p2_dpp0<0x112>(a); b += p2_dpp0<0x112>(b); c += p2_dpp0<0x112>(c); d += p2_dpp0<0x112>(d);
  a += p2_dpp0<0x114>(a); b += p2_dpp0<0x114>(b); c += p2_dpp0<0x114>(c); d += p2_dpp0<0x114>(d);
  a += p2_dpp0<0x118>(a); b += p2_dpp0<0x118>(b); c += p2_dpp0<0x118>(c); d += p2_dpp0<0x118>(d);
  p2_scan_row_carries(a, b, c, d);
}

__device__ __forceinline__ float p2_wave_sum(float v) {
  v = p2_wave_scan_incl(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ double p2_wave_sum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, P2_WAVE);
  return v;
}

// Workgroup barrier that orders LDS traffic only: outstanding global loads and stores are
// NOT waited for, so it must not be used to hand global data between lanes.
__device__ __forceinline__ void p2_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Block-wide sum of one float per thread; `red` needs >= blockDim/64 floats.
// All threads get the result.  Contains two barriers.
template <int NWAVES>
__device__ __forceinline__ float p2_block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = p2_wave_sum(v);
  p2_sync_lds();  // protect `red` from a previous use
  if (lane == 0) red[wave] = v;
  p2_sync_lds();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) s += red[w];
  return s;
}

template <int NWAVES>
__device__ __forceinline__ double p2_block_sum(double v, double* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = p2_wave_sum(v);
  p2_sync_lds();
  if (lane == 0) red[wave] = v;
  p2_sync_lds();
  double s = 0.0;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) s += red[w];
  return s;
}

// 8-byte vector view of a 1326-float row (row stride 5304 B keeps 8-byte alignment
// as long as the tensor base is 8-byte aligned; the host wrappers check that).
__device__ __forceinline__ const float2* p2_row2(const float* base, int64_t row) {
  return reinterpret_cast<const float2*>(base + row * P2_H);
}
__device__ __forceinline__ float2* p2_row2(float* base, int64_t row) {
  return reinterpret_cast<float2*>(base + row * P2_H);
}

namespace p2 {
// two floats as one 32-bit word of bfloat16 / float16 (element type codes of the C ABI: 0 float32, 1 bfloat16, 2 float16)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {   // round to nearest even, like torch
  // the part's own two-wide conversion (one instruction; spelled out in integer arithmetic it is about ten)
  typedef float p2_float2v __attribute__((ext_vector_type(2)));
  typedef __bf16 p2_bf16x2 __attribute__((ext_vector_type(2)));
  const p2_float2v v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, p2_bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16(float a, float b) {
  const _Float16 x = (_Float16)a, y = (_Float16)b;
  return (uint32_t)__builtin_bit_cast(uint16_t, x) | ((uint32_t)__builtin_bit_cast(uint16_t, y) << 16);
}
}  // namespace p2

static inline bool p2_aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
static inline bool p2_aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
