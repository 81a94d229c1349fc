/* 7-card hand ranker, plain-C restatement.  TEST INFRASTRUCTURE ONLY: the
 * product library never links or calls this file.
 *
 * Restates src/p2/env/rules.py:136-299 (create_comparison_vector), the nibble
 * packing of rules.py:111-112 / :406-407 and the card-id evaluator of
 * src/p2/env/rules_triton.py:414-581 on bit masks:
 *   - ranks ordered by (count desc, rank desc), padded with absent ranks
 *     high -> low, feed quads / full house / trips / two pair / pair / high;
 *   - straight flush reports the HIGHEST window, straight the LOWEST;
 *   - window w (0..9) covers ranks w-1..w+3, ace doubling as rank -1.
 * Pinned by tests/golden/ranker_golden.npz (written by running the reference's
 * rules.py), tests/golden/ranker_cards_golden.npz (written by running the reference's
 * card-id kernel on hands that repeat a card), the exhaustive C(52,7) category
 * histogram and std_eval.c.
 */
#include <stdint.h>
#include <string.h>

typedef struct {
    uint32_t suit[4];   /* rank masks per suit; card-id input: the SUM of the cards' rank bits (a repeated card carries) */
    uint32_t quads, trips, pairs, singles; /* rank masks by multiplicity */
} p2o_hand;

static inline int hi_bit(uint32_t x) { return 31 - __builtin_clz(x); }

static inline int pop_top(p2o_hand *h, uint32_t *zeros, int *count) {
    uint32_t *sel;
    if (h->quads) { sel = &h->quads; *count = 4; }
    else if (h->trips) { sel = &h->trips; *count = 3; }
    else if (h->pairs) { sel = &h->pairs; *count = 2; }
    else if (h->singles) { sel = &h->singles; *count = 1; }
    else { sel = zeros; *count = 0; }
    int idx = *sel ? hi_bit(*sel) : 0;
    *sel &= ~(1u << idx);
    return idx;
}

static inline uint32_t windows(uint32_t m13) {
    /* bit w set iff ranks w-1..w+3 all present (ace low for w = 0) */
    uint32_t ext = (m13 << 1) | ((m13 >> 12) & 1u);
    return ext & (ext >> 1) & (ext >> 2) & (ext >> 3) & (ext >> 4) & 0x3FFu;
}

static inline int32_t pack6(int f0, int f1, int f2, int f3, int f4, int f5) {
    return (int32_t)((f0 << 20) | (f1 << 16) | (f2 << 12) | (f3 << 8) | (f4 << 4) | f5);
}

/* flush_first != 0: flush suit = first suit with >= 5 ranks (rules_triton.py);
 * flush_first == 0: suit with the most ranks, first on ties (rules.py:217-219) */
static int32_t score(p2o_hand h, int flush_first) {
    uint32_t rank_mask = h.quads | h.trips | h.pairs | h.singles;
    uint32_t zeros = 0x1FFFu & ~(h.quads | h.trips | h.pairs | h.singles);
    int idx[5], cnt[5];
    for (int i = 0; i < 5; ++i) idx[i] = pop_top(&h, &zeros, &cnt[i]);

    int32_t best = pack6(1, idx[0], idx[1], idx[2], idx[3], idx[4]);
    int32_t s;
    if (cnt[0] >= 2) { s = pack6(2, idx[0], idx[1], idx[2], idx[3], 0); if (s > best) best = s; }
    if (cnt[0] >= 2 && cnt[1] >= 2) { s = pack6(3, idx[0], idx[1], idx[2], 0, 0); if (s > best) best = s; }
    if (cnt[0] >= 3) { s = pack6(4, idx[0], idx[1], idx[2], 0, 0); if (s > best) best = s; }
    uint32_t sw = windows(rank_mask);
    if (sw) { s = pack6(5, __builtin_ctz(sw), 0, 0, 0, 0); if (s > best) best = s; }
    int fs = -1, fc = 0;
    for (int k = 0; k < 4; ++k) {
        int c = __builtin_popcount(h.suit[k]);
        if (flush_first) { if (fs < 0 && c >= 5) { fs = k; fc = c; } }
        else if (c > fc) { fs = k; fc = c; }
    }
    if (fs >= 0 && fc >= 5) {
        uint32_t m = h.suit[fs]; int f[5];
        for (int i = 0; i < 5; ++i) { f[i] = hi_bit(m); m &= ~(1u << f[i]); }
        s = pack6(6, f[0], f[1], f[2], f[3], f[4]); if (s > best) best = s;
    }
    if (cnt[0] >= 3 && cnt[1] >= 2) { s = pack6(7, idx[0], idx[1], 0, 0, 0); if (s > best) best = s; }
    if (cnt[0] >= 4) { s = pack6(8, idx[0], idx[1], 0, 0, 0); if (s > best) best = s; }
    uint32_t sfw = windows(h.suit[0]) | windows(h.suit[1]) | windows(h.suit[2]) | windows(h.suit[3]);
    if (sfw) { s = pack6(9, hi_bit(sfw), 0, 0, 0, 0); if (s > best) best = s; }
    return best;
}

static inline p2o_hand from_suits(const uint32_t s[4]) {
    p2o_hand h; memcpy(h.suit, s, sizeof(h.suit));
    uint32_t a = s[0] ^ s[1], b = s[0] & s[1], c = s[2] ^ s[3], d = s[2] & s[3];
    uint32_t bit0 = a ^ c, carry = a & c, bit1 = b ^ d ^ carry, bit2 = b & d;
    h.quads = bit2; h.trips = bit0 & bit1; h.pairs = bit1 & ~bit0; h.singles = bit0 & ~bit1 & ~bit2;
    return h;
}

/* planes: [n, 52] bytes (0/1), suit-major like [4,13]; semantics of rules.py */
void p2o_rank_planes(const uint8_t *planes, int64_t n, int32_t *out) {
    for (int64_t i = 0; i < n; ++i) {
        uint32_t s[4] = {0, 0, 0, 0};
        const uint8_t *p = planes + i * 52;
        for (int c = 0; c < 52; ++c) if (p[c]) s[c / 13] |= 1u << (c % 13);
        out[i] = score(from_suits(s), 0);
    }
}

/* cards: [n, k] int16 ids (negative = absent); semantics of rules_triton.py:414-446: a repeated id
 * counts again for the multiplicities, and a suit mask is the integer sum of its cards' rank bits
 * (tl.sum, :421-425), so a repeated card carries into the next higher bit of its suit's mask */
void p2o_rank_cards(const int16_t *cards, int64_t n, int k, int32_t *out) {
    for (int64_t i = 0; i < n; ++i) {
        p2o_hand h; memset(&h, 0, sizeof(h));
        uint32_t seen = 0, p2 = 0, p3 = 0, p4 = 0;
        for (int j = 0; j < k; ++j) {
            int c = cards[i * k + j];
            if (c < 0) continue;
            uint32_t bit = 1u << (c % 13);
            h.suit[c / 13] += bit;
            p4 |= p3 & bit; p3 |= p2 & bit; p2 |= seen & bit; seen |= bit;
        }
        h.quads = p4; h.trips = p3 & ~p4; h.pairs = p2 & ~p3; h.singles = seen & ~p2;
        out[i] = score(h, 1);
    }
}

/* Category histogram (packed >> 20) over all C(52,7) hands; hist[10]. */
void p2o_hist_all7(uint64_t *hist) {
    uint64_t total[10] = {0};
#pragma omp parallel for schedule(dynamic, 1)
    for (int c0 = 0; c0 < 46; ++c0) {
        uint64_t loc[10] = {0};
        for (int c1 = c0 + 1; c1 < 47; ++c1)
        for (int c2 = c1 + 1; c2 < 48; ++c2)
        for (int c3 = c2 + 1; c3 < 49; ++c3)
        for (int c4 = c3 + 1; c4 < 50; ++c4)
        for (int c5 = c4 + 1; c5 < 51; ++c5)
        for (int c6 = c5 + 1; c6 < 52; ++c6) {
            int cs[7] = {c0, c1, c2, c3, c4, c5, c6};
            uint32_t s[4] = {0, 0, 0, 0};
            for (int j = 0; j < 7; ++j) s[cs[j] / 13] |= 1u << (cs[j] % 13);
            loc[score(from_suits(s), 0) >> 20]++;
        }
#pragma omp critical
        for (int t = 0; t < 10; ++t) total[t] += loc[t];
    }
    for (int t = 0; t < 10; ++t) hist[t] = total[t];
}
