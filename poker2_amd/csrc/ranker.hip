// 7-card hand ranker: one lane per hand, integer only.
//
// Replaces the Triton programs of src/p2/env/rules_triton.py (:584-632, one
// program per hand) and the torch op chain of src/p2/env/rules.py:136-299.
// A hand is four 13-bit suit masks plus four rank masks by multiplicity
// (quads / trips / pairs / singles); every category score is a 24-bit packed
// integer (type nibble + five kicker nibbles) and the result is their maximum,
// which is the reference's "row with the highest type" because the type sits
// in the top nibble.
#pragma once
#include "common.h"

namespace p2 {

struct Hand {
  uint32_t s0, s1, s2, s3;               // suit masks: bit r = the suit holds rank r (card-id input: the SUM of the
                                         // cards' rank bits, so a repeated card carries into the next bit)
  uint32_t quads, trips, pairs, singles;  // rank masks by multiplicity
};

__host__ __device__ __forceinline__ int hi_bit(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return 31 - __clz((int)x);
#else
  return 31 - __builtin_clz(x);
#endif
}
__host__ __device__ __forceinline__ int lo_bit(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __ffs((int)x) - 1;
#else
  return __builtin_ctz(x);
#endif
}
__host__ __device__ __forceinline__ int popc(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __popc(x);
#else
  return __builtin_popcount(x);
#endif
}

// bit w (0..9) set iff ranks w-1..w+3 are all present, ace doubling as rank -1
__host__ __device__ __forceinline__ uint32_t windows(uint32_t m) {
  uint32_t e = (m << 1) | ((m >> 12) & 1u);
  return e & (e >> 1) & (e >> 2) & (e >> 3) & (e >> 4) & 0x3FFu;
}

__host__ __device__ __forceinline__ Hand hand_from_suits(uint32_t s0, uint32_t s1, uint32_t s2,
                                                         uint32_t s3) {
  // bit-sliced count of the four suit bits per rank
  uint32_t a = s0 ^ s1, b = s0 & s1, c = s2 ^ s3, d = s2 & s3;
  uint32_t bit0 = a ^ c, carry = a & c, bit1 = b ^ d ^ carry, bit2 = b & d;
  Hand h;
  h.s0 = s0; h.s1 = s1; h.s2 = s2; h.s3 = s3;
  h.quads = bit2;
  h.trips = bit0 & bit1;
  h.pairs = bit1 & ~bit0;
  h.singles = bit0 & ~bit1 & ~bit2;
  return h;
}

// Card-id insertion as the reference's card kernel does it: a repeated id counts again towards the
// multiplicities (rules_triton.py:431-440), and a suit's mask is the integer SUM of its cards' rank
// bits (:421-425), so the second copy of a card carries into the next higher bit instead of being
// absorbed.  Hands of distinct cards — everything the search looks at — are not affected; the combos
// that hold a board card in rank_hands_triton (:120-148) are, and score as the reference scores them.
struct CardAcc {
  uint32_t s0 = 0, s1 = 0, s2 = 0, s3 = 0, seen = 0, p2 = 0, p3 = 0, p4 = 0;
  __host__ __device__ __forceinline__ void add(int card) {
    // ids outside 0..51 keep a rank in 0..12 and match no suit
    const uint32_t c = (uint32_t)card;
    const uint32_t suit = c / 13u;
    const uint32_t rank = c - suit * 13u;
    const uint32_t bit = 1u << rank;
    s0 += (suit == 0) ? bit : 0u;
    s1 += (suit == 1) ? bit : 0u;
    s2 += (suit == 2) ? bit : 0u;
    s3 += (suit == 3) ? bit : 0u;
    p4 |= p3 & bit;
    p3 |= p2 & bit;
    p2 |= seen & bit;
    seen |= bit;
  }
  __host__ __device__ __forceinline__ Hand finish() const {
    Hand h;
    h.s0 = s0; h.s1 = s1; h.s2 = s2; h.s3 = s3;
    h.quads = p4;
    h.trips = p3 & ~p4;
    h.pairs = p2 & ~p3;
    h.singles = seen & ~p2;
    return h;
  }
};

__host__ __device__ __forceinline__ int32_t pack6(int f0, int f1, int f2, int f3, int f4, int f5) {
  return (f0 << 20) | (f1 << 16) | (f2 << 12) | (f3 << 8) | (f4 << 4) | f5;
}
__host__ __device__ __forceinline__ int32_t imax(int32_t a, int32_t b) { return a > b ? a : b; }

// flush_first: flush suit = first suit with >= 5 ranks (rules_triton.py:229-242);
// otherwise the suit with the most ranks, first on ties (rules.py:215-219).
// The two agree whenever at most 9 cards are present.
__host__ __device__ __forceinline__ int32_t score_hand(Hand h, bool flush_first) {
  const uint32_t rank_mask = h.quads | h.trips | h.pairs | h.singles;   // ranks present, whatever the suit masks carry
  uint32_t q = h.quads, t = h.trips, p = h.pairs, s = h.singles;
  uint32_t z = 0x1FFFu & ~(q | t | p | s);
  int idx[5], cnt[5];
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    // highest rank of the highest non-empty multiplicity class; absent ranks last
    uint32_t sel = q ? q : (t ? t : (p ? p : (s ? s : z)));
    int c = q ? 4 : (t ? 3 : (p ? 2 : (s ? 1 : 0)));
    int k = sel ? hi_bit(sel) : 0;
    uint32_t clr = ~(1u << k);
    if (q) q &= clr; else if (t) t &= clr; else if (p) p &= clr; else if (s) s &= clr; else z &= clr;
    idx[i] = k;
    cnt[i] = c;
  }
  int32_t best = pack6(1, idx[0], idx[1], idx[2], idx[3], idx[4]);
  const bool c0_2 = cnt[0] >= 2, c0_3 = cnt[0] >= 3, c0_4 = cnt[0] >= 4, c1_2 = cnt[1] >= 2;
  best = imax(best, c0_2 ? pack6(2, idx[0], idx[1], idx[2], idx[3], 0) : 0);
  best = imax(best, (c0_2 && c1_2) ? pack6(3, idx[0], idx[1], idx[2], 0, 0) : 0);
  best = imax(best, c0_3 ? pack6(4, idx[0], idx[1], idx[2], 0, 0) : 0);
  const uint32_t sw = windows(rank_mask);
  best = imax(best, sw ? pack6(5, lo_bit(sw), 0, 0, 0, 0) : 0);
  const int n0 = popc(h.s0), n1 = popc(h.s1), n2 = popc(h.s2), n3 = popc(h.s3);
  uint32_t fm = 0;
  if (flush_first) {
    fm = (n0 >= 5) ? h.s0 : (n1 >= 5) ? h.s1 : (n2 >= 5) ? h.s2 : (n3 >= 5) ? h.s3 : 0u;
  } else {
    int bn = n0; fm = h.s0;
    if (n1 > bn) { bn = n1; fm = h.s1; }
    if (n2 > bn) { bn = n2; fm = h.s2; }
    if (n3 > bn) { bn = n3; fm = h.s3; }
    if (bn < 5) fm = 0;
  }
  if (fm) {
    int f[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) { f[i] = hi_bit(fm); fm &= ~(1u << f[i]); }
    best = imax(best, pack6(6, f[0], f[1], f[2], f[3], f[4]));
  }
  best = imax(best, (c0_3 && c1_2) ? pack6(7, idx[0], idx[1], 0, 0, 0) : 0);
  best = imax(best, c0_4 ? pack6(8, idx[0], idx[1], 0, 0, 0) : 0);
  const uint32_t sfw = windows(h.s0) | windows(h.s1) | windows(h.s2) | windows(h.s3);
  best = imax(best, sfw ? pack6(9, hi_bit(sfw), 0, 0, 0, 0) : 0);
  return best;
}

// ---- kernels ------------------------------------------------------------------

// Copy a contiguous byte range [byte0, byte0+nbytes) of global memory into LDS
// with dword loads; byte0 is a multiple of 4, the source base is 4-byte aligned,
// bytes past `total_bytes` are never read.
__device__ __forceinline__ void stage_bytes(const uint8_t* __restrict__ g, int64_t byte0, int nbytes,
                                            int64_t total_bytes, uint32_t* lds) {
  const uint32_t* g32 = reinterpret_cast<const uint32_t*>(g + byte0);
  const int ndw = (nbytes + 3) >> 2;
  for (int i = threadIdx.x; i < ndw; i += blockDim.x) {
    int64_t b = byte0 + 4 * (int64_t)i;
    uint32_t v = 0;
    if (b + 4 <= total_bytes) {
      v = g32[i];
    } else {
      for (int k = 0; k < 4; ++k)
        if (b + k < total_bytes) v |= (uint32_t)g[b + k] << (8 * k);
    }
    lds[i] = v;
  }
}

template <typename T>
__device__ __forceinline__ int lds_card(const uint32_t* lds, int elem) {
  return (int)reinterpret_cast<const T*>(lds)[elem];
}

constexpr int RANK_BLOCK = 256;

// cards [n, hands_per_row, 7] of T (int8 / int16); out[n] = packed score
// (hands_per_row == 1) or sign(score0 - score1) (hands_per_row == 2).
template <typename T, int HANDS>
__global__ __launch_bounds__(RANK_BLOCK) void rank_cards_small_kernel(const T* __restrict__ cards, int64_t n,
                                                                       int32_t* __restrict__ out) {
  constexpr int ROW_ELEMS = 7 * HANDS;
  constexpr int BLOCK_BYTES = RANK_BLOCK * ROW_ELEMS * (int)sizeof(T);
  __shared__ uint32_t lds[BLOCK_BYTES / 4];
  const int64_t row0 = (int64_t)blockIdx.x * RANK_BLOCK;
  const int64_t total_bytes = n * ROW_ELEMS * (int64_t)sizeof(T);
  const int64_t byte0 = row0 * ROW_ELEMS * (int64_t)sizeof(T);
  int nbytes = BLOCK_BYTES;
  if (byte0 + nbytes > total_bytes) nbytes = (int)(total_bytes - byte0);
  stage_bytes(reinterpret_cast<const uint8_t*>(cards), byte0, nbytes, total_bytes, lds);
  __syncthreads();
  const int64_t row = row0 + threadIdx.x;
  if (row >= n) return;
  int32_t sc[HANDS];
#pragma unroll
  for (int hnd = 0; hnd < HANDS; ++hnd) {
    CardAcc acc;
#pragma unroll
    for (int j = 0; j < 7; ++j) acc.add(lds_card<T>(lds, threadIdx.x * ROW_ELEMS + hnd * 7 + j));
    sc[hnd] = score_hand(acc.finish(), true);
  }
  if (HANDS == 1) out[row] = sc[0];
  else out[row] = (sc[0] > sc[HANDS - 1]) ? 1 : ((sc[0] < sc[HANDS - 1]) ? -1 : 0);
}

// 8-byte ids: read straight from global (compatibility path for torch.long input)
template <int HANDS>
__global__ __launch_bounds__(RANK_BLOCK) void rank_cards_i64_kernel(const int64_t* __restrict__ cards, int64_t n,
                                                                     int32_t* __restrict__ out) {
  const int64_t row = (int64_t)blockIdx.x * RANK_BLOCK + threadIdx.x;
  if (row >= n) return;
  int32_t sc[HANDS];
#pragma unroll
  for (int hnd = 0; hnd < HANDS; ++hnd) {
    CardAcc acc;
#pragma unroll
    for (int j = 0; j < 7; ++j) acc.add((int)cards[(row * HANDS + hnd) * 7 + j]);
    sc[hnd] = score_hand(acc.finish(), true);
  }
  if (HANDS == 1) out[row] = sc[0];
  else out[row] = (sc[0] > sc[HANDS - 1]) ? 1 : ((sc[0] < sc[HANDS - 1]) ? -1 : 0);
}

// planes [n, HANDS, 52] bytes (non-zero = card present), suit-major.
// The 52-byte rows of a workgroup's 256 hands are fetched with coalesced dword loads into LDS;
// a lane then reads its own 13 dwords (stride 13: conflict free) and folds each into four card
// bits with one multiply.
template <int HANDS>
__global__ __launch_bounds__(RANK_BLOCK) void rank_planes_kernel(const uint8_t* __restrict__ planes, int64_t n,
                                                                  int32_t* __restrict__ out, int flush_first) {
  constexpr int ROW_DW = 13 * HANDS;  // 52 bytes = 13 dwords per hand; rows are dword aligned
  __shared__ uint32_t buf[RANK_BLOCK * ROW_DW];
  const int64_t row0 = (int64_t)blockIdx.x * RANK_BLOCK;
  const int64_t rows_here = (n - row0) < RANK_BLOCK ? (n - row0) : RANK_BLOCK;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(planes) + row0 * ROW_DW;
  const int total = (int)rows_here * ROW_DW;
  for (int i = threadIdx.x; i < total; i += RANK_BLOCK) buf[i] = src[i];
  __syncthreads();
  if ((int64_t)threadIdx.x >= rows_here) return;
  int32_t sc[HANDS];
#pragma unroll
  for (int hnd = 0; hnd < HANDS; ++hnd) {
    const uint32_t* mine = buf + threadIdx.x * ROW_DW + hnd * 13;
    uint64_t cards = 0;
#pragma unroll
    for (int w = 0; w < 13; ++w) {
      const uint32_t v = mine[w];
      // bit 7 of every non-zero byte, moved to bit 0, then the four flags gathered into a nibble
      const uint32_t nz = ((((v & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | v) >> 7) & 0x01010101u;
      const uint32_t nib = (nz * 0x01020408u) >> 24;
      cards |= (uint64_t)(nib & 0xFu) << (4 * w);
    }
    sc[hnd] = score_hand(hand_from_suits((uint32_t)(cards & 0x1FFFu), (uint32_t)((cards >> 13) & 0x1FFFu),
                                         (uint32_t)((cards >> 26) & 0x1FFFu), (uint32_t)((cards >> 39) & 0x1FFFu)),
                         flush_first != 0);
  }
  const int64_t row = row0 + threadIdx.x;
  if (HANDS == 1) out[row] = sc[0];
  else out[row] = (sc[0] > sc[HANDS - 1]) ? 1 : ((sc[0] < sc[HANDS - 1]) ? -1 : 0);
}

template <int HANDS>
static int launch_rank_cards(const void* cards, int elem_size, int64_t n, int32_t* out, hipStream_t st) {
  if (n < 0 || (n > 0 && (!cards || !out))) return P2_EINVAL;
  if (n == 0) return 0;
  if (!p2_aligned4(out)) return P2_EINVAL;
  const unsigned grid = (unsigned)((n + RANK_BLOCK - 1) / RANK_BLOCK);
  if (elem_size == 1) {
    if (!p2_aligned4(cards)) return P2_EINVAL;
    hipLaunchKernelGGL((rank_cards_small_kernel<int8_t, HANDS>), dim3(grid), dim3(RANK_BLOCK), 0, st,
                       (const int8_t*)cards, n, out);
  } else if (elem_size == 2) {
    if (!p2_aligned4(cards)) return P2_EINVAL;
    hipLaunchKernelGGL((rank_cards_small_kernel<int16_t, HANDS>), dim3(grid), dim3(RANK_BLOCK), 0, st,
                       (const int16_t*)cards, n, out);
  } else if (elem_size == 8) {
    if (!p2_aligned8(cards)) return P2_EINVAL;
    hipLaunchKernelGGL((rank_cards_i64_kernel<HANDS>), dim3(grid), dim3(RANK_BLOCK), 0, st,
                       (const int64_t*)cards, n, out);
  } else {
    return P2_EINVAL;
  }
  P2_LAUNCH_CHECK();
  return 0;
}

}  // namespace p2

extern "C" {

int p2hip_rank7_cards(const void* cards, int elem_size, int64_t n, int32_t* out, void* stream) {
  return p2::launch_rank_cards<1>(cards, elem_size, n, out, (hipStream_t)stream);
}

int p2hip_compare7_cards(const void* cards, int elem_size, int64_t n, int32_t* out, void* stream) {
  return p2::launch_rank_cards<2>(cards, elem_size, n, out, (hipStream_t)stream);
}

int p2hip_rank7_planes(const uint8_t* planes, int64_t n, int32_t* out, int flush_first, void* stream) {
  if (n < 0 || (n > 0 && (!planes || !out))) return P2_EINVAL;
  if (n == 0) return 0;
  if (!p2_aligned4(planes) || !p2_aligned4(out)) return P2_EINVAL;
  const unsigned grid = (unsigned)((n + p2::RANK_BLOCK - 1) / p2::RANK_BLOCK);
  hipLaunchKernelGGL((p2::rank_planes_kernel<1>), dim3(grid), dim3(p2::RANK_BLOCK), 0, (hipStream_t)stream,
                     planes, n, out, flush_first);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_compare7_planes(const uint8_t* planes, int64_t n, int32_t* out, int flush_first, void* stream) {
  if (n < 0 || (n > 0 && (!planes || !out))) return P2_EINVAL;
  if (n == 0) return 0;
  if (!p2_aligned4(planes) || !p2_aligned4(out)) return P2_EINVAL;
  const unsigned grid = (unsigned)((n + p2::RANK_BLOCK - 1) / p2::RANK_BLOCK);
  hipLaunchKernelGGL((p2::rank_planes_kernel<2>), dim3(grid), dim3(p2::RANK_BLOCK), 0, (hipStream_t)stream,
                     planes, n, out, flush_first);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
