/* Independent textbook best-5-of-7 evaluator used ONLY to check the oracle
 * ranker where the reference is standard poker.  TEST INFRASTRUCTURE ONLY.
 * It shares no code or idea with ranker.c: it enumerates the 21 five-card
 * subsets, classifies each with counting arrays and keeps the maximum of
 * (category, tie-break ranks).  Categories use the reference numbering
 * (9 straight flush .. 1 high card, rules.py:17-28).
 */
#include <stdint.h>

static uint32_t eval5(const int *c) {
    int cnt[13] = {0}, suit_cnt[4] = {0};
    for (int i = 0; i < 5; ++i) { cnt[c[i] % 13]++; suit_cnt[c[i] / 13]++; }
    int flush = 0;
    for (int s = 0; s < 4; ++s) if (suit_cnt[s] == 5) flush = 1;
    /* ranks sorted by (count desc, rank desc) */
    int order[5], n = 0;
    for (int want = 4; want >= 1; --want)
        for (int r = 12; r >= 0; --r)
            if (cnt[r] == want) order[n++] = r;
    int distinct = n;
    int straight_high = -1;
    if (distinct == 5) {
        int hi = order[0], lo = order[4];
        if (hi - lo == 4) straight_high = hi;
        else if (hi == 12 && order[1] == 3 && lo == 0) straight_high = 3; /* wheel */
    }
    int cat;
    if (straight_high >= 0 && flush) cat = 9;
    else if (cnt[order[0]] == 4) cat = 8;
    else if (cnt[order[0]] == 3 && distinct == 2) cat = 7;
    else if (flush) cat = 6;
    else if (straight_high >= 0) cat = 5;
    else if (cnt[order[0]] == 3) cat = 4;
    else if (cnt[order[0]] == 2 && cnt[order[1]] == 2) cat = 3;
    else if (cnt[order[0]] == 2) cat = 2;
    else cat = 1;
    uint32_t key = (uint32_t)cat << 20;
    if (cat == 9 || cat == 5) return key | ((uint32_t)straight_high << 16);
    for (int i = 0; i < distinct; ++i) key |= (uint32_t)order[i] << (4 * (4 - i));
    return key;
}

/* out[i] = max over 5-subsets; comparable between hands (bigger = stronger) */
void p2o_std_best5(const int16_t *cards, int64_t n, uint32_t *out) {
    for (int64_t i = 0; i < n; ++i) {
        const int16_t *h = cards + i * 7;
        uint32_t best = 0;
        for (int a = 0; a < 7; ++a)
            for (int b = a + 1; b < 7; ++b) {
                int c5[5], k = 0;
                for (int j = 0; j < 7; ++j) if (j != a && j != b) c5[k++] = h[j];
                uint32_t v = eval5(c5);
                if (v > best) best = v;
            }
        out[i] = best;
    }
}
