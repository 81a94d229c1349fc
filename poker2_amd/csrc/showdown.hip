// River showdown: per-board strength tables (built once per subgame) and the
// per-iteration blocker-corrected EV of both players.
//
// Replaces rank_hands (src/p2/env/rules.py:66-133, rules_triton.py:120-148),
// _init_hand_rank_data (src/p2/search/cfr_evaluator.py:406-482) and
// _showdown_value / _showdown_value_both (:484-601).  The reference prefix-sums a
// [M,1327,52] tensor per call; here each card keeps only its own 51 combos in
// strength order, so one call is three short LDS scans per player:
//   P[k]        prefix of the villain range in strength order (k = 0..1326)
//   Pc[c][j]    prefix over the j weakest of the 51 combos holding card c
//   hero (a,b) at sorted position k with tie group [L,R):
//     win = P[L] - Pc[a][iLa] - Pc[b][iLb]
//     tie = P[R]-P[L] - (Pc[a][iRa]-Pc[a][iLa]) - (Pc[b][iRb]-Pc[b][iLb]) + v[k]
//     den = max(1 - Pc[a][51] - Pc[b][51] + v[k], 1e-8)
// where iLa = how many of card a's combos lie strictly below the tie group, etc.
#pragma once
#include "common.h"
#include "ranker.hip"

namespace p2 {

// ---- per-board table layout (bytes) ------------------------------------------
// perm     u16[1326]  sorted position -> combo index; bit 15 = combo blocked by the board
// lr       u16[1326][2]  tie group [L, R) of the sorted position
// cidx     u8 [1326][4]  iLa, iRa, iLb, iRb (see above)
// clist    u16[52][51]   sorted positions of the combos holding card c, ascending;
//                        all 0xFFFF for a board card (its column is masked out)
constexpr int SD_OFF_PERM = 0;
constexpr int SD_OFF_LR = SD_OFF_PERM + P2_H * 2;
constexpr int SD_OFF_CIDX = SD_OFF_LR + P2_H * 4;
constexpr int SD_OFF_CLIST = SD_OFF_CIDX + P2_H * 4;
constexpr int SD_TABLE_USED = SD_OFF_CLIST + P2_CARDS * 51 * 2;  // 18564
constexpr int SD_TABLE_BYTES = 18688;                             // padded to 256 B
static_assert(SD_TABLE_USED <= SD_TABLE_BYTES, "table layout");

constexpr int SD_BLOCK = 256;
constexpr int SD_WAVES = SD_BLOCK / 64;
constexpr int SORT_N = 2048;

// Block-wide bitonic sort of 2048 uint64 keys in LDS, ascending.
__device__ void bitonic_sort_2048(unsigned long long* keys) {
  for (int k = 2; k <= SORT_N; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      __syncthreads();
      for (int i = threadIdx.x; i < SORT_N; i += SD_BLOCK) {
        const int ixj = i ^ j;
        if (ixj > i) {
          const unsigned long long x = keys[i], y = keys[ixj];
          const bool up = (i & k) == 0;
          if ((x > y) == up) { keys[i] = y; keys[ixj] = x; }
        }
      }
    }
  }
  __syncthreads();
}

// Per-card lists: clist[c][j] = sorted position of the j-th weakest of the 51 combos holding card
// c, found by counting how many of the other 50 lie below (positions are distinct).  Ends with a
// barrier.
__device__ __forceinline__ void fill_card_lists(const uint16_t* pos_of, uint16_t (*clist)[52]) {
  for (int e = threadIdx.x; e < P2_CARDS * 51; e += SD_BLOCK) {
    const int c = e / 51, j = e % 51;
    const int x = j < c ? j : j + 1;
    const int mine = pos_of[p2_combo_index(x < c ? x : c, x < c ? c : x)];
    int below = 0;
    for (int jj = 0; jj < 51; ++jj) {
      const int y = jj < c ? jj : jj + 1;
      below += pos_of[p2_combo_index(y < c ? y : c, y < c ? c : y)] < mine ? 1 : 0;
    }
    clist[c][below] = (uint16_t)mine;
  }
  __syncthreads();
}

// How many entries of one card's list lie strictly below sorted position `bound`.
__device__ __forceinline__ int card_list_below(const uint16_t* list51, int bound) {
  int lo = 0, hi = 51;
  while (lo < hi) { const int mid = (lo + hi) >> 1; if ((int)list51[mid] < bound) lo = mid + 1; else hi = mid; }
  return lo;
}

template <typename T>
__device__ __forceinline__ int board_card(const void* boards, int64_t m, int j) {
  return (int)reinterpret_cast<const T*>(boards)[m * 5 + j];
}

// One workgroup per board.
//   mode 0: score = union of hole and board planes (a combo touching the board is a
//           6-card hand), rules.py:86-102; ranks_out = dense 1-based group ids
//   mode 1: score from the 7 card ids, hole cards first (a repeated id counts twice),
//           rules_triton.py:139-148; ranks_out = packed scores
// ranks_out [M,1326] int32, order_out [M,1326] int64 (stable ascending argsort) and
// table_out are each optional.
__global__ __launch_bounds__(SD_BLOCK) void showdown_setup_kernel(const void* __restrict__ boards, int elem_size,
                                                                   int mode, int32_t* __restrict__ ranks_out,
                                                                   int64_t* __restrict__ order_out,
                                                                   uint8_t* __restrict__ table_out) {
  __shared__ unsigned long long keys[SORT_N];
  __shared__ uint16_t pos_of[P2_H];       // combo -> sorted position
  __shared__ uint16_t clist[P2_CARDS][52];
  __shared__ int scan_tmp[SD_WAVES];
  __shared__ int bcards[5];
  const int64_t m = blockIdx.x;
  if (threadIdx.x < 5) {
    int c = elem_size == 1 ? board_card<int8_t>(boards, m, threadIdx.x)
          : elem_size == 2 ? board_card<int16_t>(boards, m, threadIdx.x)
          : elem_size == 4 ? board_card<int32_t>(boards, m, threadIdx.x)
                           : board_card<int64_t>(boards, m, threadIdx.x);
    bcards[threadIdx.x] = c;
  }
  __syncthreads();
  uint32_t bs[4] = {0, 0, 0, 0};
  unsigned long long board_bits = 0;
  for (int j = 0; j < 5; ++j) {
    const uint32_t c = (uint32_t)bcards[j];
    if (c < 52u) { bs[c / 13u] |= 1u << (c % 13u); board_bits |= 1ull << c; }
  }
  for (int h = threadIdx.x; h < SORT_N; h += SD_BLOCK) {
    unsigned long long key = ~0ull;
    if (h < P2_H) {
      const int a = p2_combo.a[h], b = p2_combo.b[h];
      int32_t sc;
      if (mode == 0) {
        uint32_t s[4] = {bs[0], bs[1], bs[2], bs[3]};
        s[a / 13] |= 1u << (a % 13);
        s[b / 13] |= 1u << (b % 13);
        sc = score_hand(hand_from_suits(s[0], s[1], s[2], s[3]), false);
      } else {
        CardAcc acc;
        acc.add(a);
        acc.add(b);
        for (int j = 0; j < 5; ++j)
          if ((uint32_t)bcards[j] < 52u) acc.add(bcards[j]);
        sc = score_hand(acc.finish(), true);
      }
      key = ((unsigned long long)(uint32_t)sc << 11) | (unsigned long long)h;
    }
    keys[h] = key;
  }
  bitonic_sort_2048(keys);  // ties resolve by combo index: a stable argsort

  for (int k = threadIdx.x; k < P2_H; k += SD_BLOCK) {
    const unsigned long long key = keys[k];
    const int h = (int)(key & 2047ull);
    pos_of[h] = (uint16_t)k;
    if (order_out) order_out[m * P2_H + k] = h;
    if (mode == 1 && ranks_out) ranks_out[m * P2_H + h] = (int32_t)(key >> 11);
  }
  __syncthreads();

  // dense group ids (mode 0): 1 + number of group starts at sorted positions 1..k
  if (mode == 0 && ranks_out) {
    // each thread owns 6 consecutive sorted positions (256*6 = 1536 >= 1326)
    const int k0 = threadIdx.x * 6;
    int flags[6], local = 0;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      const int k = k0 + i;
      flags[i] = (k > 0 && k < P2_H && (keys[k] >> 11) != (keys[k - 1] >> 11)) ? 1 : 0;
      local += flags[i];
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = local;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int o = __shfl_up(incl, off, 64);
      if (lane >= off) incl += o;
    }
    if (lane == 63) scan_tmp[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += scan_tmp[w];
    int run = base + incl - local;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      const int k = k0 + i;
      run += flags[i];
      if (k < P2_H) ranks_out[m * P2_H + (int)(keys[k] & 2047ull)] = run + 1;
    }
  }
  if (!table_out) return;
  uint16_t* t_perm = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_PERM);
  uint16_t* t_lr = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_LR);

  fill_card_lists(pos_of, clist);
  uint16_t* t_clist = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_CLIST);
  for (int e = threadIdx.x; e < P2_CARDS * 51; e += SD_BLOCK) {
    const int c = e / 51, j = e % 51;
    const bool on_board = (board_bits >> c) & 1ull;
    t_clist[e] = on_board ? (uint16_t)0xFFFF : clist[c][j];
  }
  uint8_t* t_cidx = table_out + m * SD_TABLE_BYTES + SD_OFF_CIDX;
  for (int k = threadIdx.x; k < P2_H; k += SD_BLOCK) {
    const unsigned long long key = keys[k];
    const unsigned long long sc = key >> 11;
    const int h = (int)(key & 2047ull);
    // [L, R): first position with this score, first position with a larger one
    int lo = 0, hi = k;
    while (lo < hi) { int mid = (lo + hi) >> 1; if ((keys[mid] >> 11) < sc) lo = mid + 1; else hi = mid; }
    const int L = lo;
    lo = k + 1; hi = P2_H;
    while (lo < hi) { int mid = (lo + hi) >> 1; if ((keys[mid] >> 11) <= sc) lo = mid + 1; else hi = mid; }
    const int R = lo;
    const int a = p2_combo.a[h], b = p2_combo.b[h];
    const bool blocked = ((board_bits >> a) | (board_bits >> b)) & 1ull;
    t_perm[k] = (uint16_t)(h | (blocked ? 0x8000 : 0));
    t_lr[2 * k] = (uint16_t)L;
    t_lr[2 * k + 1] = (uint16_t)R;
    t_cidx[4 * k + 0] = (uint8_t)card_list_below(clist[a], L);
    t_cidx[4 * k + 1] = (uint8_t)card_list_below(clist[a], R);
    t_cidx[4 * k + 2] = (uint8_t)card_list_below(clist[b], L);
    t_cidx[4 * k + 3] = (uint8_t)card_list_below(clist[b], R);
  }
}

// The same table from hands that are ALREADY in strength order: row m lists, per sorted position,
// the two cards of the hand (any order) and its tie group [L, R).  No board is involved, so no
// combo is flagged as blocked and no card list is masked.  The rows must list each of the 1326
// combos once; `bad[m]` is set to 1 otherwise (a card outside 0..51, a repeated combo, or a tie
// group outside 0 <= L <= k < R <= 1326) and the row's table must not be used.
__global__ __launch_bounds__(SD_BLOCK) void showdown_setup_sorted_kernel(const int32_t* __restrict__ c1,
                                                                          const int32_t* __restrict__ c2,
                                                                          const int32_t* __restrict__ L_idx,
                                                                          const int32_t* __restrict__ R_idx,
                                                                          uint8_t* __restrict__ table_out,
                                                                          int32_t* __restrict__ bad) {
  __shared__ uint16_t pos_of[P2_H];
  __shared__ uint16_t clist[P2_CARDS][52];
  __shared__ int n_bad;
  const int64_t m = blockIdx.x;
  if (threadIdx.x == 0) n_bad = 0;
  for (int h = threadIdx.x; h < P2_H; h += SD_BLOCK) pos_of[h] = 0xFFFFu;
  __syncthreads();
  uint16_t* t_perm = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_PERM);
  uint16_t* t_lr = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_LR);
  int wrong = 0;
  for (int k = threadIdx.x; k < P2_H; k += SD_BLOCK) {
    const int x = c1[m * P2_H + k], y = c2[m * P2_H + k];
    const int L = L_idx[m * P2_H + k], R = R_idx[m * P2_H + k];
    const bool ok = (uint32_t)x < 52u && (uint32_t)y < 52u && x != y && L >= 0 && L <= k && R > k && R <= P2_H;
    int h = 0;
    if (ok) {
      h = p2_combo_index(x < y ? x : y, x < y ? y : x);
      pos_of[h] = (uint16_t)k;      // a repeated combo leaves another one at 0xFFFF: counted below
    } else {
      wrong = 1;
    }
    t_perm[k] = (uint16_t)h;
    t_lr[2 * k] = (uint16_t)(ok ? L : k);
    t_lr[2 * k + 1] = (uint16_t)(ok ? R : k + 1);
  }
  __syncthreads();
  for (int h = threadIdx.x; h < P2_H; h += SD_BLOCK) wrong |= pos_of[h] == 0xFFFFu ? 1 : 0;
  if (wrong) atomicOr(&n_bad, 1);
  __syncthreads();
  if (n_bad) {                     // uniform: leave the row unusable but every table byte defined and in range
    if (threadIdx.x == 0) bad[m] = 1;
    for (int h = threadIdx.x; h < P2_H; h += SD_BLOCK) pos_of[h] = (uint16_t)h;
    __syncthreads();
  } else if (threadIdx.x == 0) {
    bad[m] = 0;
  }
  fill_card_lists(pos_of, clist);
  uint16_t* t_clist = reinterpret_cast<uint16_t*>(table_out + m * SD_TABLE_BYTES + SD_OFF_CLIST);
  for (int e = threadIdx.x; e < P2_CARDS * 51; e += SD_BLOCK) t_clist[e] = clist[e / 51][e % 51];
  uint8_t* t_cidx = table_out + m * SD_TABLE_BYTES + SD_OFF_CIDX;
  for (int k = threadIdx.x; k < P2_H; k += SD_BLOCK) {
    const int h = t_perm[k];
    const int a = p2_combo.a[h], b = p2_combo.b[h];
    const int L = t_lr[2 * k], R = t_lr[2 * k + 1];
    t_cidx[4 * k + 0] = (uint8_t)card_list_below(clist[a], L);
    t_cidx[4 * k + 1] = (uint8_t)card_list_below(clist[a], R);
    t_cidx[4 * k + 2] = (uint8_t)card_list_below(clist[b], L);
    t_cidx[4 * k + 3] = (uint8_t)card_list_below(clist[b], R);
  }
}

// ---- per-call evaluation ---------------------------------------------------------
constexpr int SD_PPT = 6;  // consecutive sorted positions per thread: 256 * 6 = 1536 >= 1326

// Row pitch of the per-card prefixes in float2.  With 52 a card's row starts 104 banks after its
// neighbour's, so cards 8 apart share their banks and the look-ups of a card's total (column 51) of 32
// lanes fall on 8 bank pairs; 53 spreads rows over all 32 pairs.
constexpr int SD_PC_STRIDE = 53;

// Everything the evaluation of one node needs in LDS.  The two heroes index every table alike
// (positions, tie groups and card lists depend on the board only), so their values sit side by
// side and one 64-bit LDS access serves both.
struct ShowdownLds {
  __align__(8) float2 v[P2_H + 2];        // .x / .y = villain-of-hero-0 / -1 range in strength order (beliefs[1] / [0] sorted)
  float2 P[P2_H + 2];                     // exclusive prefix, k = 0..1326
  float2 Pc[P2_CARDS][SD_PC_STRIDE];      // per-card exclusive prefix, Pc[c][j], j = 0..51
  float part[2][SD_WAVES];
};

// The slice of one board's table that a lane needs, kept in registers for as long as the
// board is in use (every showdown leaf of one root shares it).
struct ShowdownRegs {
  uint32_t perm[SD_PPT];   // combo index, bit 15 = blocked by the board; 0xFFFFFFFF past the end
  uint32_t lr[SD_PPT];     // L | R << 16
  uint32_t cidx[SD_PPT];   // iLa | iRa << 8 | iLb << 16 | iRb << 24
  uint32_t ab[SD_PPT];     // the combo's two cards, a | b << 8
  uint32_t clist[13];      // lane j < 51: sorted position of the j-th weakest combo of card wave + 4*i
};

struct __attribute__((packed, aligned(4))) SdU3 { uint32_t x, y, z; };

// Table slice of this lane's six consecutive sorted positions.  1326 = 221 * 6, so a lane is
// either entirely inside the table or entirely past its end and the 12 / 24 / 24 bytes it owns
// are fetched as three-dword loads (the table sections are 4-byte aligned).
// `ab_lds` (optional): a | b << 8 per combo, staged in LDS by the caller; null reads the
// constant table in global memory instead.
__device__ __forceinline__ void showdown_load_regs(const uint8_t* __restrict__ tab, ShowdownRegs& R,
                                                   const uint16_t* ab_lds = nullptr) {
  const uint16_t* clist = reinterpret_cast<const uint16_t*>(tab + SD_OFF_CLIST);
  const bool ok = threadIdx.x * SD_PPT < P2_H;
  // Lanes past the end of the table repeat lane 0's loads and drop what they get (no branch around
  // the loads, no defaults to set up): only `perm` marks them, nothing reads their lr / cidx / ab.
  const int t = ok ? (int)threadIdx.x : 0;
  const SdU3 pm = *reinterpret_cast<const SdU3*>(tab + SD_OFF_PERM + t * (SD_PPT * 2));
  const SdU3* lr = reinterpret_cast<const SdU3*>(tab + SD_OFF_LR + t * (SD_PPT * 4));
  const SdU3* cx = reinterpret_cast<const SdU3*>(tab + SD_OFF_CIDX + t * (SD_PPT * 4));
  const SdU3 l0 = lr[0], l1 = lr[1], c0 = cx[0], c1 = cx[1];
  // this lane's entry of the card lists of cards wave, wave + 4, ...: one base address, constant steps
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint16_t* mine = clist + wave * 51 + (lane < 51 ? lane : 50);
  uint32_t cl[13];
#pragma unroll
  for (int i = 0; i < 13; ++i) cl[i] = mine[i * (4 * 51)];
  const uint32_t raw[SD_PPT] = {pm.x & 0xFFFFu, pm.x >> 16, pm.y & 0xFFFFu, pm.y >> 16, pm.z & 0xFFFFu, pm.z >> 16};
  R.lr[0] = l0.x; R.lr[1] = l0.y; R.lr[2] = l0.z; R.lr[3] = l1.x; R.lr[4] = l1.y; R.lr[5] = l1.z;
  R.cidx[0] = c0.x; R.cidx[1] = c0.y; R.cidx[2] = c0.z; R.cidx[3] = c1.x; R.cidx[4] = c1.y; R.cidx[5] = c1.z;
#pragma unroll
  for (int i = 0; i < SD_PPT; ++i) {
    const int h = (int)(raw[i] & 0x7FFFu);
    R.perm[i] = ok ? raw[i] : 0xFFFFFFFFu;
    R.ab[i] = ab_lds ? (uint32_t)ab_lds[h] : ((uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8));
  }
#pragma unroll
  for (int i = 0; i < 13; ++i) R.clist[i] = lane < 51 ? cl[i] : 0xFFFFu;
}

// Gather both ranges of the node whose beliefs start at `bel` ([2,H]) into strength order:
// vk[p][i] = villain-of-hero-p mass at this lane's i-th sorted position.
__device__ __forceinline__ void showdown_gather(const float* __restrict__ bel, const ShowdownRegs& R,
                                                float (&vk)[2][SD_PPT]) {
#pragma unroll
  for (int i = 0; i < SD_PPT; ++i) {
    const bool ok = R.perm[i] != 0xFFFFFFFFu;
    const int h = (int)(R.perm[i] & 0x7FFFu);
    vk[0][i] = ok ? bel[P2_H + h] : 0.f;
    vk[1][i] = ok ? bel[h] : 0.f;
  }
}

// Showdown EV of both players from gathered ranges, written in combo order to ev ((hero 0, hero 1)
// per combo, 1326 float2 in LDS) already multiplied by mul0 / mul1 and divided by `div`; 0 for
// combos blocked by the board.  ev may be s.v (dead by the time it is written).  Uses LDS barriers
// only; the caller puts an LDS barrier before reading ev and another before the next call.
// First half of showdown_eval: sorted ranges, their prefix and the per-card prefixes into LDS.
// Ends with an LDS barrier.
__device__ __forceinline__ void showdown_scans(const float (&vk)[2][SD_PPT], const ShowdownRegs& R, ShowdownLds& s) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int k0 = threadIdx.x * SD_PPT;
  float local[2] = {0.f, 0.f}, incl[2];
#pragma unroll
  for (int i = 0; i < SD_PPT; ++i) {
    if (k0 + i < P2_H) s.v[k0 + i] = make_float2(vk[0][i], vk[1][i]);
    local[0] += vk[0][i];
    local[1] += vk[1][i];
  }
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    incl[p] = p2_wave_scan_incl(local[p]);
    if (lane == 63) s.part[p][wave] = incl[p];
  }
  p2_sync_lds();
  {
    float base0 = 0.f, base1 = 0.f;
    for (int w = 0; w < wave; ++w) { base0 += s.part[0][w]; base1 += s.part[1][w]; }
    float run0 = base0 + (incl[0] - local[0]), run1 = base1 + (incl[1] - local[1]);
#pragma unroll
    for (int i = 0; i < SD_PPT; ++i) {
      if (k0 + i <= P2_H) s.P[k0 + i] = make_float2(run0, run1);
      run0 += vk[0][i];
      run1 += vk[1][i];
    }
  }
  // per-card prefixes: one wave scan per (player, card); this wave owns cards wave, wave+4, ...
  // Both players' lists of a card share the positions, so they are scanned in lockstep, two cards at
  // a time; the lists of the next four cards are read from LDS before the current four are scanned.
  auto fetch4 = [&](int i0, float2 (&x)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j < 13 ? i0 + j : 12;
      const uint32_t pos = R.clist[i];
      const float2 y = s.v[pos < (uint32_t)P2_H ? pos : 0u];
      x[j] = pos < (uint32_t)P2_H ? y : make_float2(0.f, 0.f);
    }
  };
  auto put = [&](int i, float x0, float x1) {
    const int c = wave + 4 * i;
    if (lane < 51) s.Pc[c][lane + 1] = make_float2(x0, x1);
    if (lane == 0) s.Pc[c][0] = make_float2(0.f, 0.f);
  };
  float2 cur[4], nxt[4];
  fetch4(0, cur);
#pragma unroll
  for (int i0 = 0; i0 < 13; i0 += 4) {
    if (i0 + 4 < 13) fetch4(i0 + 4, nxt);
    if (i0 + 1 < 13) {
      p2_wave_scan_incl4(cur[0].x, cur[0].y, cur[1].x, cur[1].y);
      put(i0, cur[0].x, cur[0].y);
      put(i0 + 1, cur[1].x, cur[1].y);
    } else {
      p2_wave_scan_incl2(cur[0].x, cur[0].y);
      put(i0, cur[0].x, cur[0].y);
    }
    if (i0 + 3 < 13) {
      p2_wave_scan_incl4(cur[2].x, cur[2].y, cur[3].x, cur[3].y);
      put(i0 + 2, cur[2].x, cur[2].y);
      put(i0 + 3, cur[3].x, cur[3].y);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) cur[j] = nxt[j];
  }
  p2_sync_lds();
}

// Second half: eight 64-bit LDS reads per hand serve both players; EVs written in combo order to ev.
__device__ __forceinline__ void showdown_finish(const float (&vk)[2][SD_PPT], const ShowdownRegs& R,
                                                const ShowdownLds& s, float2* ev, float mul0, float mul1, float div) {
  const float r0 = mul0 / div, r1 = mul1 / div;  // potential / scale of the node, one division each
#pragma unroll
  for (int i = 0; i < SD_PPT; ++i) {
    if (R.perm[i] == 0xFFFFFFFFu) continue;
    const int h = (int)(R.perm[i] & 0x7FFFu);
    const bool live = !(R.perm[i] & 0x8000u);   // not blocked by the board
    const int L = (int)(R.lr[i] & 0xFFFFu), Rr = (int)(R.lr[i] >> 16);
    const int a = (int)(R.ab[i] & 0xFFu), b = (int)(R.ab[i] >> 8);
    const int iLa = (int)(R.cidx[i] & 0xFFu), iRa = (int)((R.cidx[i] >> 8) & 0xFFu);
    const int iLb = (int)((R.cidx[i] >> 16) & 0xFFu), iRb = (int)(R.cidx[i] >> 24);
    const float2 PL2 = s.P[L], PR2 = s.P[Rr];
    const float2 aL2 = s.Pc[a][iLa], aR2 = s.Pc[a][iRa], bL2 = s.Pc[b][iLb], bR2 = s.Pc[b][iRb];
    const float2 aT2 = s.Pc[a][51], bT2 = s.Pc[b][51];
    float e[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const float v0 = vk[p][i];
      const float PL = p ? PL2.y : PL2.x, PR = p ? PR2.y : PR2.x;
      const float aL = p ? aL2.y : aL2.x, aR = p ? aR2.y : aR2.x;
      const float bL = p ? bL2.y : bL2.x, bR = p ? bR2.y : bR2.x;
      const float win = PL - aL - bL;
      const float tie = (PR - PL) - (aR - aL) - (bR - bL) + v0;
      float den = 1.0f - (p ? aT2.y : aT2.x) - (p ? bT2.y : bT2.x) + v0;
      den = fmaxf(den, 1e-8f);
      // The kernel is VALU-issue bound and an IEEE division is about ten instructions, so both
      // quotients share one hardware reciprocal and are corrected by one fused residual step
      // each, which keeps x/x == 1 and 0/x == 0 exact (an all-tie board stays exactly zero).
      // a hand the board blocks goes the way of an empty denominator: every quotient 0, EV 0
      const bool valid = live && den > 1e-8f;
      const float inv = valid ? __builtin_amdgcn_rcpf(den) : 0.f;
      float wp = win * inv, tp = tie * inv;
      wp = __builtin_fmaf(__builtin_fmaf(-wp, den, win), inv, wp);
      tp = __builtin_fmaf(__builtin_fmaf(-tp, den, tie), inv, tp);
      const float lp = valid ? 1.0f - wp - tp : 0.f;
      e[p] = wp - lp;
    }
    ev[h] = make_float2(e[0] * r0, e[1] * r1);
  }
}

__device__ __forceinline__ void showdown_eval(const float (&vk)[2][SD_PPT], const ShowdownRegs& R, ShowdownLds& s,
                                              float2* ev, float mul0, float mul1, float div) {
  showdown_scans(vk, R, s);
  showdown_finish(vk, R, s, ev, mul0, mul1, div);
}

// out[n] = showdown EV of both players at node n.
//   beliefs   [M,2,H]      range pair per node
//   table_row [M] or null  row of `tables` to use for node n (null: row n)
//   potential [M,2] float  chips won by player p if he wins; scale [M]
// Workgroups walk the nodes with a grid stride; the table slice of the next node is requested
// before the scans of the current one and its ranges are gathered between the scans and the
// final pass, so the two dependent global round trips of a node overlap the LDS work of the
// previous one.
__global__ __launch_bounds__(SD_BLOCK, 3) void showdown_both_kernel(const float* __restrict__ beliefs,
                                                                     const uint8_t* __restrict__ tables,
                                                                     const int64_t* __restrict__ table_row,
                                                                     const float* __restrict__ potential,
                                                                     const float* __restrict__ scale, int64_t m,
                                                                     float* __restrict__ out) {
  __shared__ ShowdownLds s;
  __shared__ uint16_t ab_lds[P2_H];
  for (int h = threadIdx.x; h < P2_H; h += SD_BLOCK) ab_lds[h] = (uint16_t)(p2_combo.a[h] | (p2_combo.b[h] << 8));
  p2_sync_lds();
  ShowdownRegs R, Rn;
  float vk[2][SD_PPT], vkn[2][SD_PPT];
  int64_t n = blockIdx.x;
  if (n < m) {
    showdown_load_regs(tables + (table_row ? table_row[n] : n) * SD_TABLE_BYTES, Rn, ab_lds);
    showdown_gather(beliefs + n * 2 * P2_H, Rn, vkn);
  }
  for (; n < m; n += gridDim.x) {
    R = Rn;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int i = 0; i < SD_PPT; ++i) vk[p][i] = vkn[p][i];
    const int64_t nn = n + gridDim.x;
    const bool more = nn < m;
    if (more) showdown_load_regs(tables + (table_row ? table_row[nn] : nn) * SD_TABLE_BYTES, Rn, ab_lds);
    const float mul0 = potential[2 * n], mul1 = potential[2 * n + 1], div = scale[n];
    showdown_scans(vk, R, s);
    if (more) showdown_gather(beliefs + nn * 2 * P2_H, Rn, vkn);
    // the EVs go over the sorted ranges, which are dead once the card scans are done
    showdown_finish(vk, R, s, s.v, mul0, mul1, div);
    p2_sync_lds();
    float2* o0 = p2_row2(out, n * 2);
    float2* o1 = p2_row2(out, n * 2 + 1);
    for (int i = threadIdx.x; i < P2_HPAIRS; i += SD_BLOCK) {
      const float2 x = s.v[2 * i], y = s.v[2 * i + 1];   // hands 2i, 2i+1: (hero 0, hero 1) each
      o0[i] = make_float2(x.x, y.x);
      o1[i] = make_float2(x.y, y.y);
    }
    p2_sync_lds();  // the next node overwrites s.v
  }
}

}  // namespace p2

extern "C" {

int64_t p2hip_showdown_table_bytes(void) { return p2::SD_TABLE_BYTES; }

int p2hip_showdown_setup(const void* boards, int elem_size, int64_t m, int mode, int32_t* ranks_out,
                         int64_t* order_out, uint8_t* table_out, void* stream) {
  if (m < 0 || (m > 0 && !boards)) return P2_EINVAL;
  if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8) return P2_EINVAL;
  if (mode != 0 && mode != 1) return P2_EINVAL;
  if (m == 0) return 0;
  if (table_out && !p2_aligned8(table_out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::showdown_setup_kernel, dim3((unsigned)m), dim3(p2::SD_BLOCK), 0, (hipStream_t)stream,
                     boards, elem_size, mode, ranks_out, order_out, table_out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_showdown_setup_sorted(const int32_t* c1_sorted, const int32_t* c2_sorted, const int32_t* L_idx,
                                const int32_t* R_idx, int64_t m, uint8_t* table_out, int32_t* bad, void* stream) {
  if (m < 0 || m > 0x7FFFFFFF) return P2_EINVAL;
  if (m == 0) return 0;
  if (!c1_sorted || !c2_sorted || !L_idx || !R_idx || !table_out || !bad) return P2_EINVAL;
  if (!p2_aligned8(table_out) || !p2_aligned4(c1_sorted) || !p2_aligned4(c2_sorted) || !p2_aligned4(L_idx) ||
      !p2_aligned4(R_idx) || !p2_aligned4(bad))
    return P2_EINVAL;
  hipLaunchKernelGGL(p2::showdown_setup_sorted_kernel, dim3((unsigned)m), dim3(p2::SD_BLOCK), 0, (hipStream_t)stream,
                     c1_sorted, c2_sorted, L_idx, R_idx, table_out, bad);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_showdown_both(const float* beliefs, const uint8_t* tables, const int64_t* table_row,
                        const float* potential, const float* scale, int64_t m, float* out, void* stream) {
  if (m < 0 || (m > 0 && (!beliefs || !tables || !potential || !scale || !out))) return P2_EINVAL;
  if (m == 0) return 0;
  if (!p2_aligned8(tables) || !p2_aligned4(beliefs) || !p2_aligned8(out)) return P2_EINVAL;
  const int64_t cap = 256 * 3;  // three resident workgroups (43 KB of LDS each) on each of the 256 CUs
  hipLaunchKernelGGL(p2::showdown_both_kernel, dim3((unsigned)(m < cap ? m : cap)), dim3(p2::SD_BLOCK), 0,
                     (hipStream_t)stream, beliefs, tables, table_row, potential, scale, m, out);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
