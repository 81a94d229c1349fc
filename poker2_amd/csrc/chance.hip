// Single-card chance node around the leaf network: expansion of a public state's ranges over
// every card that can come next, and the mean of the network's answers.
//
// Replaces the tensor program of ChanceNodeHelper.single_card_chance_values
// (src/p2/search/chance_node_helper.py:360-479):
//   expand : for every state i and every card c not on its board, in (i, c) ascending order,
//            post[s][p][h] = pre[i][p][h] if h holds neither c nor a board card, else 0,
//            renormalised per player (uniform over the allowed hands if the sum is <= 1e-12);
//            board_samples[s] = board with c in the first empty slot; root_lookup[s] = i
//            (:394-443)
//   mean   : expected[i] = sum of hand_values over the samples of state i / their count
//            (:467-477)
// The per-sample sum of a player's masked range is T - cs[c] (T = total of the board-masked
// range, cs[c] = its mass on hands holding c), so one card-sum pass per state serves all of
// its 46-49 samples.  The expansion is a pure write stream (about 48 x 10.6 KB per state).
//
// A state's samples are one contiguous run of 2652-float blocks.  The main kernel treats the run a
// workgroup writes as a flat sequence of float4 and places its lanes on absolute 128-byte lines, so every
// wave-wide store covers whole lines (rows of 5304 bytes never start on one); the state's masked ranges
// and the hands' cards are staged in LDS and each float4 looks up its sample and hands there.  Buffers
// that are only 8-byte aligned take the row-wise float2 kernel.
#pragma once
#include <mutex>
#include "common.h"
#include "unblocked.hip"

namespace p2 {

constexpr int CH_BLOCK = 256;
constexpr int CH_PPT = 3;  // float2 pairs per thread and vector
constexpr int CH_SPLIT = 13;  // workgroups per state in the expansion (4 candidate cards each)
static_assert(P2_CARDS % CH_SPLIT == 0, "card runs");
static_assert(CH_BLOCK == UB_BLOCK, "card_sums_multi assumes the block size");

__device__ __forceinline__ int chance_board(const int64_t* __restrict__ board5, int (&cards)[5], uint64_t& bits) {
  int n = 0;
  bits = 0ull;
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    const int64_t c = board5[j];
    cards[j] = (int)c;
    if (c >= 0 && c < P2_CARDS) {
      bits |= 1ull << c;
      ++n;
    }
  }
  return n;
}

// Workgroup -> (state, run of candidate cards).  States are taken in groups of `group`; inside a
// group the order is run-major.  The row-wise kernel takes groups of 2048: workgroups in flight at one
// time then write chunks a megabyte apart (measured faster for it than neighbouring chunks), while a
// group's ranges (22 MB) stay in the last-level cache for the 13 visits they get (16384 states as one
// group: 2.61 ms; in groups of 2048: 1.85 ms).  The line kernel takes groups of 8 = the number of XCDs:
// workgroup b runs on XCD b mod 8, so the four workgroups of a state follow each other on one XCD and
// read its ranges from that XCD's L2 (3584 states: groups of 2048 392 us, of 8 375 us; 16384 states:
// 1.81 ms and 1.68 ms).
constexpr int CH_GROUP_ROWS = 2048;
constexpr int CH_GROUP_LINES = 8;

__device__ __forceinline__ bool chance_work(int64_t n, int parts, int group_size, int64_t& state, int& part) {
  const int64_t per_group = (int64_t)group_size * parts;
  const int64_t group = blockIdx.x / per_group, r = blockIdx.x - group * per_group;
  const int64_t first = group * group_size;
  const int64_t count = n - first < group_size ? n - first : group_size;   // the last group may be short
  if (r >= count * parts) return false;   // the grid is sized for full groups
  part = (int)(r / count);
  state = first + (r - part * count);
  return true;
}

// A state's share of the output buffers is samples [sample_offsets[i], sample_offsets[i + 1]).  When the
// state yields fewer samples than that (`have`: its board holds more cards than the caller's offsets
// assume, has no empty slot, or its row lies outside the table) the rest of the share is filled with
// zeros, root_lookup with the state, so that no row of the outputs is left uninitialised.  Called by the
// workgroup of the state's last part; `row_bytes` is a multiple of 8 and `rows` 8-byte aligned.
__device__ __forceinline__ void chance_fill_rest(const int64_t* __restrict__ sample_offsets, int64_t i, int have,
                                                 int64_t total_samples, void* rows, int64_t row_bytes,
                                                 int64_t* board_samples, int64_t* root_lookup) {
  const int64_t s0 = sample_offsets[i] + have;
  int64_t s1 = sample_offsets[i + 1];
  if (s1 > total_samples) s1 = total_samples;
  if (s0 < 0 || s0 >= s1) return;
  uint2* dst = reinterpret_cast<uint2*>(reinterpret_cast<char*>(rows) + s0 * row_bytes);
  const int64_t words = (s1 - s0) * (row_bytes / 8);
  for (int64_t k = threadIdx.x; k < words; k += blockDim.x) dst[k] = make_uint2(0u, 0u);
  for (int64_t k = threadIdx.x; k < (s1 - s0) * 5; k += blockDim.x)
    if (board_samples) board_samples[s0 * 5 + k] = 0;
  for (int64_t k = threadIdx.x; k < s1 - s0; k += blockDim.x) root_lookup[s0 + k] = i;
}

static inline unsigned chance_grid(int64_t n, int parts, int group_size) {
  return (unsigned)(((n + group_size - 1) / group_size) * group_size * parts);
}

__global__ __launch_bounds__(CH_BLOCK) void chance_expand_kernel(const float* __restrict__ pre_beliefs,
                                                                  const int64_t* __restrict__ root_indices,
                                                                  const int64_t* __restrict__ board,
                                                                  const int64_t* __restrict__ sample_offsets,
                                                                  int64_t source_rows, int64_t total_samples,
                                                                  float* __restrict__ post_beliefs,
                                                                  int64_t* __restrict__ board_samples,
                                                                  int64_t* __restrict__ root_lookup, int64_t n) {
  __shared__ __align__(8) float t[2][P2_H + 2];
  __shared__ double cs[2 * P2_CARDS];
  int64_t i;
  int part;
  if (!chance_work(n, CH_SPLIT, CH_GROUP_ROWS, i, part)) return;
  const int64_t root = root_indices ? root_indices[i] : i;
  const bool in_table = root >= 0 && root < source_rows;
  int bcards[5];
  uint64_t bits = 0;
  const int ncards = in_table ? chance_board(board + root * 5, bcards, bits) : 5;
  if (part == CH_SPLIT - 1)
    chance_fill_rest(sample_offsets, i, ncards < 5 ? P2_CARDS - ncards : 0, total_samples, post_beliefs,
                     2 * P2_H * (int64_t)sizeof(float), board_samples, root_lookup);
  if (!in_table) return;   // uniform per workgroup: nothing to read

  // this lane's hands: pairs k -> hands 2*idx, 2*idx+1 with idx = tid + k*256
  float v[2][CH_PPT][2];
  float uni[CH_PPT][2];   // the hand's share of the uniform fallback (0 for hands on the board)
  uint32_t ab[CH_PPT][2];
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    const bool in = idx < P2_HPAIRS;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int h = in ? 2 * idx + q : 0;
      ab[k][q] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8);
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      float2 x = make_float2(0.f, 0.f);
      if (in) x = p2_row2(pre_beliefs, root * 2 + p)[idx];
      const bool blocked0 = ((bits >> (ab[k][0] & 0xFFu)) | (bits >> (ab[k][0] >> 8))) & 1ull;
      const bool blocked1 = ((bits >> (ab[k][1] & 0xFFu)) | (bits >> (ab[k][1] >> 8))) & 1ull;
      v[p][k][0] = blocked0 ? 0.f : x.x;
      v[p][k][1] = blocked1 ? 0.f : x.y;
      if (in) reinterpret_cast<float2*>(t[p])[idx] = make_float2(v[p][k][0], v[p][k][1]);
    }
  }
  p2_sync_lds();
  card_sums_multi(t[0], P2_H + 2, 2, cs);
  const double total0 = card_total(cs), total1 = card_total(cs + P2_CARDS);

  const int remaining = P2_CARDS - ncards - 1;          // cards left for the hands of a sample
  const float uniform = 1.0f / fmaxf((float)(remaining * (remaining - 1) / 2), 1.0f);
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k)
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const bool on_board = ((bits >> (ab[k][q] & 0xFFu)) | (bits >> (ab[k][q] >> 8))) & 1ull;
      uni[k][q] = on_board ? 0.f : uniform;
    }
  // the 52 candidate cards are split into CH_SPLIT runs: short-lived workgroups with few
  // stores per lane keep the chip's write window dense (runs of 13 cards measured 514 us on
  // 3584 turn states, runs of 4 cards 435 us, single cards 782 us - the card-sum preamble is paid
  // per workgroup; re-reading the ranges from L2 per sample instead of keeping them in registers
  // measured slower than either); a sample's position counts the cards below it that are not on
  // the board
  const int c_begin = part * (P2_CARDS / CH_SPLIT), c_end = c_begin + P2_CARDS / CH_SPLIT;
  int64_t s = sample_offsets[i] + c_begin - __popcll(bits & ((1ull << c_begin) - 1ull));
  for (int c = c_begin; c < c_end; ++c) {
    if ((bits >> c) & 1ull) continue;
    // the caller sized the outputs for `total_samples`; a state with fewer cards on its board than
    // the caller assumed would run past them
    if (s < 0 || s >= total_samples || ncards >= 5) break;
    const float sum0 = (float)(total0 - cs[c]);
    const float sum1 = (float)(total1 - cs[P2_CARDS + c]);
    const bool ok0 = sum0 > 1e-12f, ok1 = sum1 > 1e-12f;
    const float inv0 = 1.0f / fmaxf(sum0, 1e-12f), inv1 = 1.0f / fmaxf(sum1, 1e-12f);
    float2* o0 = p2_row2(post_beliefs, s * 2);
    float2* o1 = p2_row2(post_beliefs, s * 2 + 1);
#pragma unroll
    for (int k = 0; k < CH_PPT; ++k) {
      const int idx = threadIdx.x + k * CH_BLOCK;
      if (idx >= P2_HPAIRS) continue;
      float r0[2], r1[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const uint32_t a = ab[k][q] & 0xFFu, b = ab[k][q] >> 8;
        const bool off = a == (uint32_t)c || b == (uint32_t)c;
        r0[q] = off ? 0.f : (ok0 ? v[0][k][q] * inv0 : uni[k][q]);
        r1[q] = off ? 0.f : (ok1 ? v[1][k][q] * inv1 : uni[k][q]);
      }
      o0[idx] = make_float2(r0[0], r0[1]);
      o1[idx] = make_float2(r1[0], r1[1]);
    }
    if (threadIdx.x < 5) {
      int64_t card = bcards[threadIdx.x];
      if ((int)threadIdx.x == ncards) card = c;
      board_samples[s * 5 + threadIdx.x] = card;
    }
    if (threadIdx.x == 0) root_lookup[s] = i;
    ++s;
  }
}

// ---- the expansion on whole 128-byte lines ------------------------------------------------------
constexpr int CH_QUADS = 2 * P2_H / 4;   // 663 float4 per state and per sample
constexpr int CH_QPT = 3;                // float4 per lane when a state is staged: 3 x 256 >= 663
constexpr int CH_MAX_RUN = 13;           // candidate cards per workgroup: 52 / parts with parts = 4 or 13
static_assert((2 * P2_H) % 4 == 0 && CH_QPT * CH_BLOCK >= CH_QUADS, "a state is a whole number of float4");

struct ChanceSample {   // what a float4 needs to know about its sample
  float inv0, inv1;     // 1 / the surviving mass of player 0 / 1, or 0 where the uniform fallback applies
  int card;
  int pad;
};

// What a sample's output row looks like.  INPUT_ROWS = false: the 2 x 1326 ranges as float32, samples back to
// back (`post_beliefs` [S, 2, 1326]).  INPUT_ROWS = true: a row of a value network's input matrix
// [S, CH_INPUT_WIDTH] in element type DT (0 float32, 1 bfloat16, 2 float16) — the ranges followed by the
// 52-entry one-hot of the sample's board (the state's cards and the dealt one) — so the network needs
// neither a concatenation nor a cast.  Either way a row is a whole number of 16-byte units and the
// samples of a workgroup are one contiguous run of units.
constexpr int CH_INPUT_WIDTH = 2 * P2_H + P2_CARDS;   // 2704
constexpr int CH_LDS_PAD = 8;                          // the unit that straddles the end of the ranges reads on
static_assert((CH_INPUT_WIDTH * 2) % 16 == 0 && (CH_INPUT_WIDTH * 4) % 16 == 0, "input rows are whole 16-byte units");

template <int DT, bool INPUT_ROWS>
__global__ __launch_bounds__(CH_BLOCK) void chance_expand_lines_kernel(const float* __restrict__ pre_beliefs,
                                                                        const int64_t* __restrict__ root_indices,
                                                                        const int64_t* __restrict__ board,
                                                                        const int64_t* __restrict__ sample_offsets,
                                                                        int64_t source_rows, int64_t total_samples,
                                                                        void* __restrict__ post_beliefs,
                                                                        int64_t* __restrict__ board_samples,
                                                                        int64_t* __restrict__ root_lookup, int64_t n,
                                                                        int parts) {
  static_assert(INPUT_ROWS || DT == 0, "plain ranges are float32");
  constexpr int UNIT = DT == 0 ? 4 : 8;                                        // elements per 16-byte unit
  constexpr int ROW_UNITS = (INPUT_ROWS ? CH_INPUT_WIDTH : 2 * P2_H) / UNIT;   // 663, 676 or 338
  __shared__ __align__(16) float t[2 * P2_H + CH_LDS_PAD];            // the state's ranges without the board's hands
  __shared__ __align__(16) uint16_t cards_of[2 * P2_H + CH_LDS_PAD];  // a | b << 8 of the hand behind every float of t
  __shared__ double cs[2 * P2_CARDS];
  __shared__ __align__(16) ChanceSample sample[CH_MAX_RUN];
  int64_t i;
  int part;
  if (!chance_work(n, parts, CH_GROUP_LINES, i, part)) return;
  const int64_t root = root_indices ? root_indices[i] : i;
  const bool in_table = root >= 0 && root < source_rows;
  int bcards[5];
  uint64_t bits = 0;
  const int ncards = in_table ? chance_board(board + root * 5, bcards, bits) : 5;
  if (part == parts - 1)
    chance_fill_rest(sample_offsets, i, ncards < 5 ? P2_CARDS - ncards : 0, total_samples, post_beliefs,
                     ROW_UNITS * 16ll, board_samples, root_lookup);
  if (ncards >= 5) return;                       // outside the table, or no empty slot: nothing to expand

  const float4* src = reinterpret_cast<const float4*>(pre_beliefs + root * (2 * P2_H));
#pragma unroll
  for (int k = 0; k < CH_QPT; ++k) {
    const int j = threadIdx.x + k * CH_BLOCK;
    if (j >= CH_QUADS) continue;
    const float4 x = src[j];
    const float xs[4] = {x.x, x.y, x.z, x.w};
    float y[4];
    uint16_t packed[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int f = 4 * j + q;
      const int h = f >= P2_H ? f - P2_H : f;
      const uint32_t a = p2_combo.a[h], b = p2_combo.b[h];
      packed[q] = (uint16_t)(a | (b << 8));
      y[q] = (((bits >> a) | (bits >> b)) & 1ull) ? 0.f : xs[q];
    }
    reinterpret_cast<float4*>(t)[j] = make_float4(y[0], y[1], y[2], y[3]);
    reinterpret_cast<uint2*>(cards_of)[j] = make_uint2((uint32_t)packed[0] | ((uint32_t)packed[1] << 16),
                                                       (uint32_t)packed[2] | ((uint32_t)packed[3] << 16));
  }
  if (threadIdx.x < CH_LDS_PAD) {
    t[2 * P2_H + threadIdx.x] = 0.f;
    cards_of[2 * P2_H + threadIdx.x] = 0;
  }
  p2_sync_lds();
  card_sums_multi(t, P2_H, 2, cs);
  const double total0 = card_total(cs), total1 = card_total(cs + P2_CARDS);

  // this workgroup's samples: the cards of its run that are not on the board, in ascending order
  const int run = P2_CARDS / parts;
  const int c_begin = part * run;
  const uint64_t run_bits = ((1ull << run) - 1ull) << c_begin;
  const uint64_t free_bits = ~bits & run_bits;
  const int64_t s_first = sample_offsets[i] + c_begin - __popcll(bits & ((1ull << c_begin) - 1ull));
  int count = __popcll(free_bits);
  // outputs are sized for total_samples: samples beyond them are not written
  if (s_first < 0) count = 0;
  else if (s_first + count > total_samples) count = (int)(total_samples > s_first ? total_samples - s_first : 0);
  if ((int)threadIdx.x < run) {
    const int c = c_begin + threadIdx.x;
    const int m = __popcll(free_bits & ((1ull << c) - 1ull));   // position among the run's samples
    if (((free_bits >> c) & 1ull) && m < count) {
      const float sum0 = (float)(total0 - cs[c]);
      const float sum1 = (float)(total1 - cs[P2_CARDS + c]);
      ChanceSample sm;
      sm.inv0 = sum0 > 1e-12f ? 1.0f / fmaxf(sum0, 1e-12f) : 0.f;
      sm.inv1 = sum1 > 1e-12f ? 1.0f / fmaxf(sum1, 1e-12f) : 0.f;
      sm.card = c;
      sm.pad = 0;
      sample[m] = sm;
    }
  }
  p2_sync_lds();
  if (count <= 0) return;

  // board_samples [S,5] and root_lookup [S]: lane 8 m + slot
  {
    const int m = threadIdx.x >> 3, slot = threadIdx.x & 7;
    if (m < count) {
      if (slot < 5) {
        int64_t card = bcards[0];
#pragma unroll
        for (int q = 1; q < 5; ++q) card = slot == q ? (int64_t)bcards[q] : card;
        if (slot == ncards) card = sample[m].card;
        if (board_samples) board_samples[(s_first + m) * 5 + slot] = card;
      } else if (slot == 5) {
        root_lookup[s_first + m] = i;
      }
    }
  }

  const int remaining = P2_CARDS - ncards - 1;          // cards left for the hands of a sample
  const float uniform = 1.0f / fmaxf((float)(remaining * (remaining - 1) / 2), 1.0f);
  uint4* out = reinterpret_cast<uint4*>(post_beliefs);
  const int64_t g0 = s_first * ROW_UNITS;                // first 16-byte unit of the workgroup
  const uint32_t units = (uint32_t)count * ROW_UNITS;    // at most 13 x 676
  // Lanes sit on absolute 128-byte lines (8 units): lane l takes units l - lead, l - lead + 256, ... of the
  // workgroup's run.  The sample m and the unit j inside its row follow by one division and then by increments
  // (a row has more than 256 units).
  static_assert(ROW_UNITS > CH_BLOCK, "one row boundary per step at most");
  const uint32_t lead = (uint32_t)(g0 & 7);
  uint32_t local = threadIdx.x >= lead ? threadIdx.x - lead : threadIdx.x - lead + CH_BLOCK;
  uint32_t m = local / ROW_UNITS, j = local - m * ROW_UNITS;
  for (; local < units; local += CH_BLOCK, j += CH_BLOCK) {
    if (j >= (uint32_t)ROW_UNITS) { j -= ROW_UNITS; ++m; }
    const ChanceSample sm = sample[m];
    float xs[UNIT];
    uint32_t pk[UNIT / 2];                               // a | b << 8 of two hands per word
#pragma unroll
    for (int u = 0; u < UNIT / 4; ++u) {
      // a unit behind the ranges (board one-hot only) reads the last padded quad: its values are not used
      const uint32_t quad = min(j * (UNIT / 4) + u, (uint32_t)(2 * P2_H + CH_LDS_PAD) / 4 - 1);
      const float4 x = reinterpret_cast<const float4*>(t)[quad];
      const uint2 c2 = reinterpret_cast<const uint2*>(cards_of)[quad];
      xs[4 * u] = x.x; xs[4 * u + 1] = x.y; xs[4 * u + 2] = x.z; xs[4 * u + 3] = x.w;
      pk[2 * u] = c2.x; pk[2 * u + 1] = c2.y;
    }
    const uint32_t e0 = UNIT * j;                        // first element of the unit in its row
    float r[UNIT];
    if (sm.inv0 != 0.f && sm.inv1 != 0.f) {
      // both players have mass left: value x 1 / mass, zero for a hand that holds the dealt card.  Two hands per
      // word: a byte of (cards ^ dealt card in every byte) is zero exactly where a card equals the dealt one.
      // Cards are below 64, so with bit 7 of every byte set first, subtracting 1 from every byte borrows from
      // no neighbour and clears bit 7 exactly in the bytes that were zero.
      const uint32_t rep = (uint32_t)sm.card * 0x01010101u;
#pragma unroll
      for (int w = 0; w < UNIT / 2; ++w) {
        // ranges end at an even element and units start at multiples of 4: both hands of a word are one player's
        const float inv = (e0 + 2 * w >= (uint32_t)P2_H) ? sm.inv1 : sm.inv0;
        const uint32_t x = pk[w] ^ rep;
        const uint32_t z = ~((x | 0x80808080u) - 0x01010101u) & 0x80808080u;
        r[2 * w] = (z & 0x00008080u) ? 0.f : xs[2 * w] * inv;
        r[2 * w + 1] = (z & 0x80800000u) ? 0.f : xs[2 * w + 1] * inv;
      }
    } else {
#pragma unroll
      for (int q = 0; q < UNIT; ++q) {
        const float inv = (e0 + q >= (uint32_t)P2_H) ? sm.inv1 : sm.inv0;
        const uint32_t cd = (pk[q / 2] >> (16 * (q & 1))) & 0xFFFFu;
        const uint32_t a = cd & 0xFFu, b = cd >> 8;
        float val = xs[q] * inv;
        if (inv == 0.f) val = (((bits >> a) | (bits >> b)) & 1ull) ? 0.f : uniform;   // no mass left: uniform
        r[q] = (a == (uint32_t)sm.card || b == (uint32_t)sm.card) ? 0.f : val;
      }
    }
    if (INPUT_ROWS && e0 + UNIT > (uint32_t)(2 * P2_H)) {
      const uint64_t dealt = bits | (1ull << sm.card);   // the sample's board as a card set
#pragma unroll
      for (int q = 0; q < UNIT; ++q)
        if (e0 + q >= (uint32_t)(2 * P2_H)) r[q] = ((dealt >> (e0 + q - 2 * P2_H)) & 1ull) ? 1.f : 0.f;
    }
    uint4 w;
    if (DT == 0) {
      w = make_uint4(__builtin_bit_cast(uint32_t, r[0]), __builtin_bit_cast(uint32_t, r[1]),
                     __builtin_bit_cast(uint32_t, r[2]), __builtin_bit_cast(uint32_t, r[3]));
    } else if (DT == 1) {
      w = make_uint4(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]), pack_bf16(r[4 % UNIT], r[5 % UNIT]),
                     pack_bf16(r[6 % UNIT], r[7 % UNIT]));
    } else {
      w = make_uint4(pack_f16(r[0], r[1]), pack_f16(r[2], r[3]), pack_f16(r[4 % UNIT], r[5 % UNIT]),
                     pack_f16(r[6 % UNIT], r[7 % UNIT]));
    }
    out[g0 + local] = w;
  }
}

// expected[i][p][h] = mean over the samples of state i.  The low bit of blockIdx.x picks the player: a workgroup walks the
// whole 5304-byte rows of one player through all samples of its state (three pairs per lane), four
// samples' rows in flight at a time.
__global__ __launch_bounds__(CH_BLOCK) void chance_mean_kernel(const float* __restrict__ hand_values,
                                                                const int64_t* __restrict__ sample_offsets,
                                                                float* __restrict__ expected) {
  const int64_t i = blockIdx.x >> 1;
  const int p = blockIdx.x & 1;
  const int64_t s0 = sample_offsets[i], s1 = sample_offsets[i + 1];
  float2 acc[CH_PPT];
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) acc[k] = make_float2(0.f, 0.f);
  int64_t s = s0;
  for (; s + 4 <= s1; s += 4) {
    float2 x[4][CH_PPT];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float2* row = p2_row2(hand_values, (s + j) * 2 + p);
#pragma unroll
      for (int k = 0; k < CH_PPT; ++k) {
        const int idx = threadIdx.x + k * CH_BLOCK;
        x[j][k] = row[idx < P2_HPAIRS ? idx : 0];
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int k = 0; k < CH_PPT; ++k) { acc[k].x += x[j][k].x; acc[k].y += x[j][k].y; }
  }
  for (; s < s1; ++s) {
    const float2* row = p2_row2(hand_values, s * 2 + p);
#pragma unroll
    for (int k = 0; k < CH_PPT; ++k) {
      const int idx = threadIdx.x + k * CH_BLOCK;
      const float2 v = row[idx < P2_HPAIRS ? idx : 0];
      acc[k].x += v.x; acc[k].y += v.y;
    }
  }
  const float count = fmaxf((float)(s1 - s0), 1.0f);
  float2* o = p2_row2(expected, i * 2 + p);
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    if (idx < P2_HPAIRS) o[idx] = make_float2(acc[k].x / count, acc[k].y / count);
  }
}

// ---- three-card (flop) chance node ------------------------------------------------------
// flop_chance_values (src/p2/search/chance_node_helper.py:219-357): every state is expanded over
// a list of candidate flops (the canonical ones, or a sample of them); a hand survives a flop
// if it holds none of its three cards, the survivors are renormalised (uniform over them if the
// sum is <= 1e-12).  By inclusion-exclusion the surviving mass of a range is
//   T - cs[a] - cs[b] - cs[c] + t[ab] + t[ac] + t[bc]
// so again one card-sum pass per state serves all of its flops.  out is [n, flops, 2, H].
__global__ __launch_bounds__(CH_BLOCK) void flop_expand_kernel(const float* __restrict__ pre_beliefs,
                                                                const int64_t* __restrict__ root_indices,
                                                                const int64_t* __restrict__ flops, int64_t n_flops,
                                                                float* __restrict__ out) {
  __shared__ __align__(8) float t[2][P2_H + 2];
  __shared__ double cs[2 * P2_CARDS];
  const int64_t i = blockIdx.x;
  const int64_t root = root_indices ? root_indices[i] : i;
  float v[2][CH_PPT][2];
  uint32_t ab[CH_PPT][2];
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    const bool in = idx < P2_HPAIRS;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int h = in ? 2 * idx + q : 0;
      ab[k][q] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8);
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      float2 x = make_float2(0.f, 0.f);
      if (in) {
        x = p2_row2(pre_beliefs, root * 2 + p)[idx];
        reinterpret_cast<float2*>(t[p])[idx] = x;
      }
      v[p][k][0] = x.x;
      v[p][k][1] = x.y;
    }
  }
  p2_sync_lds();
  card_sums_multi(t[0], P2_H + 2, 2, cs);
  const double total[2] = {card_total(cs), card_total(cs + P2_CARDS)};
  const float uniform = 1.0f / (float)(49 * 48 / 2);   // hands left once three cards are out
  // blockIdx.y takes a contiguous run of flops: one contiguous piece of the output per workgroup
  const int64_t per = (n_flops + gridDim.y - 1) / gridDim.y;
  const int64_t f_end = (blockIdx.y + 1) * per < n_flops ? (blockIdx.y + 1) * per : n_flops;
  for (int64_t f = blockIdx.y * per; f < f_end; ++f) {
    int c[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) c[j] = (int)flops[f * 3 + j];
    bool valid = true;
#pragma unroll
    for (int j = 0; j < 3; ++j) valid = valid && c[j] >= 0 && c[j] < P2_CARDS;
    valid = valid && c[0] != c[1] && c[0] != c[2] && c[1] != c[2];
    float inv[2];
    bool ok[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      double sum = 0.0;
      if (valid) {
        sum = total[p];
#pragma unroll
        for (int j = 0; j < 3; ++j) sum -= cs[p * P2_CARDS + c[j]];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          const int x = c[j], y = c[(j + 1) % 3];
          sum += (double)t[p][p2_combo_index(x < y ? x : y, x < y ? y : x)];
        }
      }
      const float sf = (float)sum;
      ok[p] = sf > 1e-12f;
      inv[p] = 1.0f / fmaxf(sf, 1e-12f);
    }
    float2* o0 = p2_row2(out, ((int64_t)i * n_flops + f) * 2);
    float2* o1 = p2_row2(out, ((int64_t)i * n_flops + f) * 2 + 1);
#pragma unroll
    for (int k = 0; k < CH_PPT; ++k) {
      const int idx = threadIdx.x + k * CH_BLOCK;
      if (idx >= P2_HPAIRS) continue;
      float r0[2], r1[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int a = (int)(ab[k][q] & 0xFFu), b = (int)(ab[k][q] >> 8);
        const bool off = !valid || a == c[0] || a == c[1] || a == c[2] || b == c[0] || b == c[1] || b == c[2];
        r0[q] = off ? 0.f : (ok[0] ? v[0][k][q] * inv[0] : uniform);
        r1[q] = off ? 0.f : (ok[1] ? v[1][k][q] * inv[1] : uniform);
      }
      o0[idx] = make_float2(r0[0], r0[1]);
      o1[idx] = make_float2(r1[0], r1[1]);
    }
  }
}

// The flop expansion on whole 128-byte lines: same scheme as chance_expand_lines_kernel.  out is one
// run of 2652-float blocks in (state, flop) order; a workgroup writes `run` consecutive flops of a state.
constexpr int FL_MAX_RUN = 16;

struct FlopSample {
  float inv0, inv1;    // 1 / surviving mass, or 0 where the uniform fallback applies
  uint32_t cards;      // c0 | c1 << 8 | c2 << 16, or 0xFFFFFFFF for a flop that is not three distinct cards
  uint32_t pad;
};

__global__ __launch_bounds__(CH_BLOCK) void flop_expand_lines_kernel(const float* __restrict__ pre_beliefs,
                                                                      const int64_t* __restrict__ root_indices,
                                                                      const int64_t* __restrict__ flops,
                                                                      int64_t n_flops, float* __restrict__ out,
                                                                      int64_t n, int run, int parts) {
  __shared__ __align__(16) float t[2 * P2_H];
  __shared__ __align__(16) uint16_t cards_of[2 * P2_H];
  __shared__ double cs[2 * P2_CARDS];
  __shared__ __align__(16) FlopSample sample[FL_MAX_RUN];
  int64_t i;
  int part;
  if (!chance_work(n, parts, CH_GROUP_LINES, i, part)) return;
  const int64_t root = root_indices ? root_indices[i] : i;
  const float4* src = reinterpret_cast<const float4*>(pre_beliefs + root * (2 * P2_H));
#pragma unroll
  for (int k = 0; k < CH_QPT; ++k) {
    const int j = threadIdx.x + k * CH_BLOCK;
    if (j >= CH_QUADS) continue;
    reinterpret_cast<float4*>(t)[j] = src[j];
    uint32_t packed[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int f = 4 * j + q;
      const int h = f >= P2_H ? f - P2_H : f;
      packed[q] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8);
    }
    reinterpret_cast<uint2*>(cards_of)[j] = make_uint2(packed[0] | (packed[1] << 16), packed[2] | (packed[3] << 16));
  }
  p2_sync_lds();
  card_sums_multi(t, P2_H, 2, cs);
  const double total[2] = {card_total(cs), card_total(cs + P2_CARDS)};

  const int64_t f_begin = (int64_t)part * run;
  const int count = (int)(n_flops - f_begin < run ? n_flops - f_begin : run);
  if ((int)threadIdx.x < count) {
    const int64_t f = f_begin + threadIdx.x;
    int c[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) c[j] = (int)flops[f * 3 + j];
    bool valid = true;
#pragma unroll
    for (int j = 0; j < 3; ++j) valid = valid && c[j] >= 0 && c[j] < P2_CARDS;
    valid = valid && c[0] != c[1] && c[0] != c[2] && c[1] != c[2];
    FlopSample sm;
    sm.cards = valid ? ((uint32_t)c[0] | ((uint32_t)c[1] << 8) | ((uint32_t)c[2] << 16)) : 0xFFFFFFFFu;
    sm.pad = 0;
    float inv[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      double sum = 0.0;
      if (valid) {
        sum = total[p];
#pragma unroll
        for (int j = 0; j < 3; ++j) sum -= cs[p * P2_CARDS + c[j]];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          const int x = c[j], y = c[(j + 1) % 3];
          sum += (double)t[p * P2_H + p2_combo_index(x < y ? x : y, x < y ? y : x)];
        }
      }
      const float sf = (float)sum;
      inv[p] = sf > 1e-12f ? 1.0f / fmaxf(sf, 1e-12f) : 0.f;
    }
    sm.inv0 = inv[0];
    sm.inv1 = inv[1];
    sample[threadIdx.x] = sm;
  }
  p2_sync_lds();
  if (count <= 0) return;

  const float uniform = 1.0f / (float)(49 * 48 / 2);   // hands left once three cards are out
  float4* o = reinterpret_cast<float4*>(out);
  const int64_t g0 = (i * n_flops + f_begin) * CH_QUADS, g1 = g0 + (int64_t)count * CH_QUADS;
  for (int64_t g = (g0 & ~7ll) + threadIdx.x; g < g1; g += CH_BLOCK) {
    if (g < g0) continue;
    const uint32_t local = (uint32_t)(g - g0);
    const uint32_t m = local / CH_QUADS, j = local - m * CH_QUADS;
    const FlopSample sm = sample[m];
    const float4 x = reinterpret_cast<const float4*>(t)[j];
    const uint2 pk = reinterpret_cast<const uint2*>(cards_of)[j];
    const float xs[4] = {x.x, x.y, x.z, x.w};
    const uint32_t cd[4] = {pk.x & 0xFFFFu, pk.x >> 16, pk.y & 0xFFFFu, pk.y >> 16};
    const uint32_t c0 = sm.cards & 0xFFu, c1 = (sm.cards >> 8) & 0xFFu, c2 = (sm.cards >> 16) & 0xFFu;
    const bool valid = sm.cards != 0xFFFFFFFFu;
    float r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float inv = (4 * j + q >= (uint32_t)P2_H) ? sm.inv1 : sm.inv0;
      const uint32_t a = cd[q] & 0xFFu, b = cd[q] >> 8;
      const bool off = !valid || a == c0 || a == c1 || a == c2 || b == c0 || b == c1 || b == c2;
      r[q] = off ? 0.f : (inv == 0.f ? uniform : xs[q] * inv);
    }
    o[g] = make_float4(r[0], r[1], r[2], r[3]);
  }
}

// out[i][p][h] (+)= sum_f weight[f] * mean_q hand_values[i][f][p][perms[q][h]]
// (the suit-orbit mean of _avg_over_perms, chance_node_helper.py:18-28, and the weighted sum over
// flops, :352-357).  The permutations of a call are the same for all of its flops (the reference draws
// them once per chunk of flops, chance_node_helper.py:318-329), and the gather is linear, so
//   sum_f w[f] * mean_q hv[f][perm_q[h]]  =  mean_q Y[perm_q[h]]   with   Y[j] = sum_f w[f] * hv[f][j]:
// a workgroup takes one (state, player) and one contiguous share of the flops, adds the weighted rows of its
// share hand by hand in fp64 registers - a pure read stream, CH_ROWS rows in flight per lane - and applies the
// permutations ONCE, to the sums staged in LDS, instead of once per row.  With more than one share the
// workgroups write partial results that perm_reduce_kernel adds in a fixed order.
constexpr int CH_MAX_PERMS = 24;
constexpr int CH_ROWS = 4;   // rows requested together
__global__ __launch_bounds__(CH_BLOCK) void perm_mean_kernel(const float* __restrict__ hand_values,
                                                              const int16_t* __restrict__ perms, int n_perms,
                                                              const float* __restrict__ weight, int64_t n_flops,
                                                              int64_t flops_per_share, int accumulate,
                                                              float* __restrict__ dst, int64_t dst_share_stride) {
  __shared__ double y[P2_H + 2];
  const int64_t i = blockIdx.x >> 1;
  const int p = blockIdx.x & 1;
  const int64_t f0 = (int64_t)blockIdx.y * flops_per_share;
  const int64_t f1 = f0 + flops_per_share < n_flops ? f0 + flops_per_share : n_flops;
  double acc[CH_PPT][2];
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) acc[k][0] = acc[k][1] = 0.0;
  // rows beyond the share's end repeat its last row with weight 0: straight-line loads, no branch per row
  float2 cur[CH_ROWS][CH_PPT], nxt[CH_ROWS][CH_PPT];
  auto fetch = [&](int64_t f, float2 (&r)[CH_ROWS][CH_PPT]) {
#pragma unroll
    for (int j = 0; j < CH_ROWS; ++j) {
      const int64_t fj = f + j < f1 ? f + j : f1 - 1;
      const float2* src = p2_row2(hand_values, ((int64_t)i * n_flops + fj) * 2 + p);
#pragma unroll
      for (int k = 0; k < CH_PPT; ++k) {
        const int idx = threadIdx.x + k * CH_BLOCK;
        r[j][k] = src[idx < P2_HPAIRS ? idx : 0];
      }
    }
  };
  if (f0 < f1) fetch(f0, cur);
  for (int64_t f = f0; f < f1; f += CH_ROWS) {
    if (f + CH_ROWS < f1) fetch(f + CH_ROWS, nxt);
#pragma unroll
    for (int j = 0; j < CH_ROWS; ++j) {
      const double w = f + j < f1 ? (double)weight[f + j] : 0.0;
#pragma unroll
      for (int k = 0; k < CH_PPT; ++k) {
        acc[k][0] += w * (double)cur[j][k].x;   // the product of two floats is exact in fp64
        acc[k][1] += w * (double)cur[j][k].y;
      }
    }
#pragma unroll
    for (int j = 0; j < CH_ROWS; ++j)
#pragma unroll
      for (int k = 0; k < CH_PPT; ++k) cur[j][k] = nxt[j][k];
  }
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    if (idx < P2_HPAIRS) {
      y[2 * idx] = acc[k][0];
      y[2 * idx + 1] = acc[k][1];
    }
  }
  p2_sync_lds();
  const double inv_perms = 1.0 / (double)n_perms;
  float2* o = p2_row2(dst + (int64_t)blockIdx.y * dst_share_stride, i * 2 + p);
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    if (idx >= P2_HPAIRS) continue;
    double s0 = 0.0, s1 = 0.0;
    for (int q = 0; q < n_perms; ++q) {
      const uint32_t e = reinterpret_cast<const uint32_t*>(perms + (int64_t)q * P2_H)[idx];   // two hands per dword
      s0 += y[e & 0xFFFFu];
      s1 += y[e >> 16];
    }
    const float2 prev = accumulate ? o[idx] : make_float2(0.f, 0.f);
    o[idx] = make_float2(prev.x + (float)(s0 * inv_perms), prev.y + (float)(s1 * inv_perms));
  }
}

// out (+)= sum over shares of partial[share], shares added in ascending order.
__global__ __launch_bounds__(CH_BLOCK) void perm_reduce_kernel(const float2* __restrict__ partial, int shares,
                                                                int64_t npairs, int accumulate,
                                                                float2* __restrict__ out) {
  const int64_t e = (int64_t)blockIdx.x * CH_BLOCK + threadIdx.x;
  if (e >= npairs) return;
  float2 s = accumulate ? out[e] : make_float2(0.f, 0.f);
  for (int j = 0; j < shares; ++j) {
    const float2 v = partial[(int64_t)j * npairs + e];
    s.x += v.x;
    s.y += v.y;
  }
  out[e] = s;
}

// ---- mean over the whole suit orbit ------------------------------------------------------------
// With all 24 suit permutations the mean of hv[perm_q[h]] over q is the mean of hv over the orbit of
// h (every orbit member is hit 24 / |orbit| times), and the orbits are the 169 classes of starting
// hands: 13 pairs (6 hands each), 78 suited (4), 78 offsuit (12).  So one accumulator per class
// replaces 24 look-ups per hand and flop.
constexpr int ORB_CLASSES = 169;
constexpr int ORB_MAX = 12;
struct P2OrbitTable {
  int16_t member[ORB_CLASSES][ORB_MAX];   // hands of the class, ascending; -1 past its size
  uint8_t size[ORB_CLASSES];
  uint8_t cls[P2_H];                       // class of every hand
  constexpr P2OrbitTable() : member(), size(), cls() {
    for (int c = 0; c < ORB_CLASSES; ++c) {
      size[c] = 0;
      for (int j = 0; j < ORB_MAX; ++j) member[c][j] = -1;
    }
    int h = 0;
    for (int a = 0; a < P2_CARDS; ++a) {
      for (int b = a + 1; b < P2_CARDS; ++b, ++h) {
        const int ra = a % 13, rb = b % 13, sa = a / 13, sb = b / 13;
        const int lo = ra < rb ? ra : rb, hi = ra < rb ? rb : ra;
        const int pair_index = lo * (25 - lo) / 2 + (hi - lo - 1);   // 0..77 over rank pairs lo < hi
        const int c = ra == rb ? ra : (sa == sb ? 13 + pair_index : 91 + pair_index);
        cls[h] = (uint8_t)c;
        member[c][size[c]] = (int16_t)h;
        size[c] = (uint8_t)(size[c] + 1);
      }
    }
  }
};
__device__ const P2OrbitTable p2_orbit = P2OrbitTable();

// dst[i][p][h] (+)= sum_f weight[f] * (mean of hand_values[i][f][p] over the orbit class of h).
// Workgroup layout and the share / workspace scheme are those of perm_mean_kernel.
__global__ __launch_bounds__(CH_BLOCK) void orbit_mean_kernel(const float* __restrict__ hand_values,
                                                               const float* __restrict__ weight, int64_t n_flops,
                                                               int64_t flops_per_share, int accumulate,
                                                               float* __restrict__ dst, int64_t dst_share_stride) {
  __shared__ __align__(8) float rows[2][P2_H + 2];
  __shared__ float class_acc[ORB_CLASSES];
  const int64_t i = blockIdx.x >> 1;
  const int p = blockIdx.x & 1;
  const int64_t f0 = (int64_t)blockIdx.y * flops_per_share;
  const int64_t f1 = f0 + flops_per_share < n_flops ? f0 + flops_per_share : n_flops;
  const int c = threadIdx.x;                 // lanes 0..168 own one class each
  int mem[ORB_MAX];
  float inv_size = 0.f;
#pragma unroll
  for (int j = 0; j < ORB_MAX; ++j) mem[j] = c < ORB_CLASSES ? (int)p2_orbit.member[c][j] : -1;
  if (c < ORB_CLASSES) inv_size = 1.0f / (float)p2_orbit.size[c];
  double acc = 0.0;
  float2 next[CH_PPT];
  auto fetch = [&](int64_t f) {
    const float2* src = p2_row2(hand_values, ((int64_t)i * n_flops + f) * 2 + p);
#pragma unroll
    for (int k = 0; k < CH_PPT; ++k) {
      const int idx = threadIdx.x + k * CH_BLOCK;
      next[k] = idx < P2_HPAIRS ? src[idx] : make_float2(0.f, 0.f);
    }
  };
  if (f0 < f1) fetch(f0);
  int buf = 0;
  for (int64_t f = f0; f < f1; ++f, buf ^= 1) {
    float* row = rows[buf];
#pragma unroll
    for (int k = 0; k < CH_PPT; ++k) {
      const int idx = threadIdx.x + k * CH_BLOCK;
      if (idx < P2_HPAIRS) reinterpret_cast<float2*>(row)[idx] = next[k];
    }
    if (f + 1 < f1) fetch(f + 1);
    p2_sync_lds();   // row f is complete; the other buffer was consumed before this barrier
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < ORB_MAX; ++j)
      if (mem[j] >= 0) s += row[mem[j]];
    acc += (double)(weight[f] * (s * inv_size));
  }
  if (c < ORB_CLASSES) class_acc[c] = (float)acc;
  p2_sync_lds();
  float2* o = p2_row2(dst + (int64_t)blockIdx.y * dst_share_stride, i * 2 + p);
#pragma unroll
  for (int k = 0; k < CH_PPT; ++k) {
    const int idx = threadIdx.x + k * CH_BLOCK;
    if (idx >= P2_HPAIRS) continue;
    const float2 prev = accumulate ? o[idx] : make_float2(0.f, 0.f);
    o[idx] = make_float2(prev.x + class_acc[p2_orbit.cls[2 * idx]], prev.y + class_acc[p2_orbit.cls[2 * idx + 1]]);
  }
}

}  // namespace p2

extern "C" {

int p2hip_chance_expand(const float* pre_beliefs, const int64_t* root_indices, const int64_t* board, int64_t n,
                        const int64_t* sample_offsets, int64_t source_rows, int64_t total_samples,
                        float* post_beliefs, int64_t* board_samples, int64_t* root_lookup, void* stream) {
  if (n < 0 || source_rows < 0 || total_samples < 0) return P2_EINVAL;
  if (n == 0) return 0;
  if (!pre_beliefs || !board || !sample_offsets || !post_beliefs || !board_samples || !root_lookup) return P2_EINVAL;
  if (!p2_aligned8(pre_beliefs) || !p2_aligned8(post_beliefs)) return P2_EINVAL;
  if (n > 0x7FFFFFFF / p2::CH_SPLIT - p2::CH_GROUP_ROWS) return P2_EINVAL;
  const bool wide = ((reinterpret_cast<uintptr_t>(pre_beliefs) | reinterpret_cast<uintptr_t>(post_beliefs)) & 15u) == 0;
  if (wide) {
    // runs of 13 cards = 4 workgroups per state (3584 states: 375 us, in runs of 4 cards 465 us; 333 states:
    // 37 and 42 us); runs of 4 cards only where there would be fewer workgroups than the chip takes at once
    const int parts = n >= 256 ? 4 : p2::CH_SPLIT;
    hipLaunchKernelGGL((p2::chance_expand_lines_kernel<0, false>), dim3(p2::chance_grid(n, parts, p2::CH_GROUP_LINES)),
                       dim3(p2::CH_BLOCK), 0, (hipStream_t)stream, pre_beliefs, root_indices, board, sample_offsets,
                       source_rows, total_samples, (void*)post_beliefs, board_samples, root_lookup, n, parts);
    P2_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(p2::chance_expand_kernel, dim3(p2::chance_grid(n, p2::CH_SPLIT, p2::CH_GROUP_ROWS)), dim3(p2::CH_BLOCK), 0,
                     (hipStream_t)stream, pre_beliefs, root_indices, board, sample_offsets, source_rows,
                     total_samples, post_beliefs, board_samples, root_lookup, n);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_chance_expand_input(const float* pre_beliefs, const int64_t* root_indices, const int64_t* board, int64_t n,
                              const int64_t* sample_offsets, int64_t source_rows, int64_t total_samples,
                              void* input_rows, int dtype, int64_t* board_samples, int64_t* root_lookup, void* stream) {
  if (n < 0 || source_rows < 0 || total_samples < 0 || dtype < 0 || dtype > 2) return P2_EINVAL;
  if (n == 0) return 0;
  if (!pre_beliefs || !board || !sample_offsets || !input_rows || !root_lookup) return P2_EINVAL;
  if (((reinterpret_cast<uintptr_t>(pre_beliefs) | reinterpret_cast<uintptr_t>(input_rows)) & 15u) != 0) return P2_EINVAL;
  if (n > 0x7FFFFFFF / p2::CH_SPLIT - p2::CH_GROUP_ROWS) return P2_EINVAL;
  const int parts = n >= 256 ? 4 : p2::CH_SPLIT;
  const dim3 grid(p2::chance_grid(n, parts, p2::CH_GROUP_LINES)), block(p2::CH_BLOCK);
#define P2_EXPAND_INPUT(DT)                                                                                      \
  hipLaunchKernelGGL((p2::chance_expand_lines_kernel<DT, true>), grid, block, 0, (hipStream_t)stream, pre_beliefs, \
                     root_indices, board, sample_offsets, source_rows, total_samples, input_rows, board_samples,  \
                     root_lookup, n, parts)
  if (dtype == 0) P2_EXPAND_INPUT(0);
  else if (dtype == 1) P2_EXPAND_INPUT(1);
  else P2_EXPAND_INPUT(2);
#undef P2_EXPAND_INPUT
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_chance_mean(const float* hand_values, const int64_t* sample_offsets, int64_t n, float* expected,
                      void* stream) {
  if (n < 0) return P2_EINVAL;
  if (n == 0) return 0;
  if (!hand_values || !sample_offsets || !expected) return P2_EINVAL;
  if (!p2_aligned8(hand_values) || !p2_aligned8(expected)) return P2_EINVAL;
  if (n > 0x3FFFFFFF) return P2_EINVAL;
  // the two players of a state on neighbouring workgroups: together they read the state's samples as one
  // contiguous run (3584 turn states: 345 -> 328 us against all of player 0's workgroups before player 1's)
  hipLaunchKernelGGL(p2::chance_mean_kernel, dim3((unsigned)(2 * n)), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                     hand_values, sample_offsets, expected);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_flop_expand(const float* pre_beliefs, const int64_t* root_indices, int64_t n, const int64_t* flops,
                      int64_t n_flops, float* out, void* stream) {
  if (n < 0 || n_flops < 0) return P2_EINVAL;
  if (n == 0 || n_flops == 0) return 0;
  if (!pre_beliefs || !flops || !out || !p2_aligned8(pre_beliefs) || !p2_aligned8(out)) return P2_EINVAL;
  if (n > 0x7FFFFFFF) return P2_EINVAL;
  const bool wide = ((reinterpret_cast<uintptr_t>(pre_beliefs) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  if (wide) {
    // eight flops per workgroup (1024 states x 256 flops: 4 per workgroup 645 us, 8: 525 us, 16: 530 us; the
    // row-wise kernel 585-625 us), four where eight would leave fewer than a thousand workgroups
    const int run = n * ((n_flops + 7) / 8) >= 1024 ? 8 : 4;
    static_assert(8 <= p2::FL_MAX_RUN, "run length");
    const int64_t parts = (n_flops + run - 1) / run;
    const int64_t groups = (n + p2::CH_GROUP_LINES - 1) / p2::CH_GROUP_LINES;
    if (parts > 0x7FFFFFFF || groups * p2::CH_GROUP_LINES * parts > 0x7FFFFFFF) return P2_EINVAL;
    hipLaunchKernelGGL(p2::flop_expand_lines_kernel, dim3(p2::chance_grid(n, (int)parts, p2::CH_GROUP_LINES)),
                       dim3(p2::CH_BLOCK), 0, (hipStream_t)stream, pre_beliefs, root_indices, flops, n_flops, out, n,
                       run, (int)parts);
    P2_LAUNCH_CHECK();
    return 0;
  }
  // row-wise kernel, about four flops per workgroup: fewer make the per-workgroup card-sum preamble dominate
  // (1024 states x 256 flops: 16 per workgroup 874 us, 4: 658 us, 1: 1096 us)
  const int64_t want = (n_flops + 3) / 4;
  const unsigned split = (unsigned)(want < 65535 ? want : 65535);
  hipLaunchKernelGGL(p2::flop_expand_kernel, dim3((unsigned)n, split), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                     pre_beliefs, root_indices, flops, n_flops, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_perm_mean(const float* hand_values, int64_t n, int64_t n_flops, const int16_t* perms, int n_perms,
                    const float* weight, int accumulate, float* out, float* workspace, int shares, void* stream) {
  if (n < 0 || n_flops < 0 || n_perms < 1 || n_perms > p2::CH_MAX_PERMS || shares < 1) return P2_EINVAL;
  if (n == 0) return 0;
  if (!hand_values || !perms || !weight || !out || !p2_aligned8(hand_values) || !p2_aligned8(out)) return P2_EINVAL;
  if (((uintptr_t)perms & 3) != 0) return P2_EINVAL;
  if (n > 0x3FFFFFFF || shares > 65535) return P2_EINVAL;
  if (shares > 1 && (!workspace || !p2_aligned8(workspace))) return P2_EINVAL;
  const size_t lds = 0;
  const int64_t per_share = (n_flops + shares - 1) / shares;
  const int64_t npairs = n * 2 * P2_HPAIRS;
  if (shares == 1) {
    hipLaunchKernelGGL(p2::perm_mean_kernel, dim3((unsigned)(2 * n), 1), dim3(p2::CH_BLOCK), lds, (hipStream_t)stream,
                       hand_values, perms, n_perms, weight, n_flops, per_share, accumulate, out, (int64_t)0);
    P2_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(p2::perm_mean_kernel, dim3((unsigned)(2 * n), (unsigned)shares), dim3(p2::CH_BLOCK), lds,
                     (hipStream_t)stream, hand_values, perms, n_perms, weight, n_flops, per_share, 0, workspace,
                     npairs * 2);
  P2_LAUNCH_CHECK();
  const int64_t grid = (npairs + p2::CH_BLOCK - 1) / p2::CH_BLOCK;
  hipLaunchKernelGGL(p2::perm_reduce_kernel, dim3((unsigned)grid), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                     (const float2*)workspace, shares, npairs, accumulate, (float2*)out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_orbit_mean(const float* hand_values, int64_t n, int64_t n_flops, const float* weight, int accumulate,
                     float* out, float* workspace, int shares, void* stream) {
  if (n < 0 || n_flops < 0 || shares < 1) return P2_EINVAL;
  if (n == 0) return 0;
  if (!hand_values || !weight || !out || !p2_aligned8(hand_values) || !p2_aligned8(out)) return P2_EINVAL;
  if (n > 0x3FFFFFFF || shares > 65535) return P2_EINVAL;
  if (shares > 1 && (!workspace || !p2_aligned8(workspace))) return P2_EINVAL;
  const int64_t per_share = (n_flops + shares - 1) / shares;
  const int64_t npairs = n * 2 * P2_HPAIRS;
  if (shares == 1) {
    hipLaunchKernelGGL(p2::orbit_mean_kernel, dim3((unsigned)(2 * n), 1), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                       hand_values, weight, n_flops, per_share, accumulate, out, (int64_t)0);
    P2_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(p2::orbit_mean_kernel, dim3((unsigned)(2 * n), (unsigned)shares), dim3(p2::CH_BLOCK), 0,
                     (hipStream_t)stream, hand_values, weight, n_flops, per_share, 0, workspace, npairs * 2);
  P2_LAUNCH_CHECK();
  const int64_t grid = (npairs + p2::CH_BLOCK - 1) / p2::CH_BLOCK;
  hipLaunchKernelGGL(p2::perm_reduce_kernel, dim3((unsigned)grid), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                     (const float2*)workspace, shares, npairs, accumulate, (float2*)out);
  P2_LAUNCH_CHECK();
  return 0;
}

// ---- the suit-orbit mean for callers that cannot allocate ---------------------------------------
// Partial sums of p2hip_orbit_mean_static live in this file-scope array instead of a workspace the
// caller allocates.  Every GPU the library runs on holds its own copy at its own address until the
// process ends.  In host code the array's NAME is only a handle for hipGetSymbolAddress: kernels and
// copies take the per-device address resolved below.
#define P2_ORBIT_SCRATCH_FLOATS (4 * 1024 * 1024)   /* 16 MiB; equals P2HIP_ORBIT_SCRATCH_FLOATS of include/p2hip.h */
static __device__ __align__(256) float p2_orbit_scratch[P2_ORBIT_SCRATCH_FLOATS];

namespace p2 {
constexpr int SCRATCH_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};

// Device address of the scratch array on the CURRENT device, resolved once per device.
static int orbit_scratch_address(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= SCRATCH_MAX_DEVICES) return P2_EINVAL;
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(p2_orbit_scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace p2

int p2hip_orbit_mean_static(const float* hand_values, int64_t n, int64_t n_flops, const float* weight,
                            int accumulate, float* out, int shares, void* stream) {
  if (n < 0 || n_flops < 0 || shares < 1) return P2_EINVAL;
  if (n == 0) {
    // Set-up call: resolves this device's address of the array (the first resolution on a device may load
    // the code object and is not something to do under graph capture) and launches nothing.
    float* scratch = nullptr;
    return p2::orbit_scratch_address(&scratch);
  }
  if (!hand_values || !weight || !out || !p2_aligned8(hand_values) || !p2_aligned8(out)) return P2_EINVAL;
  if (n > 0x3FFFFFFF || shares > 65535) return P2_EINVAL;
  const int64_t per_share = (n_flops + shares - 1) / shares;
  const int64_t npairs = n * 2 * P2_HPAIRS;
  if (shares == 1) {   // no partial sums: the kernel writes the output itself
    hipLaunchKernelGGL(p2::orbit_mean_kernel, dim3((unsigned)(2 * n), 1), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                       hand_values, weight, n_flops, per_share, accumulate, out, (int64_t)0);
    P2_LAUNCH_CHECK();
    return 0;
  }
  // [shares, n, 2, H] partial sums must fit the array; refused before anything is launched
  if ((int64_t)shares * npairs * 2 > (int64_t)P2_ORBIT_SCRATCH_FLOATS) return (int)hipErrorOutOfMemory;
  float* scratch = nullptr;
  const int rc = p2::orbit_scratch_address(&scratch);
  if (rc != 0) return rc;
  // Nothing in the array has to start at zero: every (share, state, player) row the reduction reads is
  // written in full by the first kernel, also by a share that holds no flop.
  hipLaunchKernelGGL(p2::orbit_mean_kernel, dim3((unsigned)(2 * n), (unsigned)shares), dim3(p2::CH_BLOCK), 0,
                     (hipStream_t)stream, hand_values, weight, n_flops, per_share, 0, scratch, npairs * 2);
  P2_LAUNCH_CHECK();
  const int64_t grid = (npairs + p2::CH_BLOCK - 1) / p2::CH_BLOCK;
  hipLaunchKernelGGL(p2::perm_reduce_kernel, dim3((unsigned)grid), dim3(p2::CH_BLOCK), 0, (hipStream_t)stream,
                     (const float2*)scratch, shares, npairs, accumulate, (float2*)out);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
