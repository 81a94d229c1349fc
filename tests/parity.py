"""Element-wise comparison of CFR state with exemptions BY CAUSE.

The iteration is float32 with hard thresholds (regret matching falls back to the uniform policy where
the positive regrets sum to less than 1e-8; belief, average-policy and opponent-mass sums fall back
below 1e-5; the showdown divides by a compatible mass clamped at 1e-8) and with differences of
nearly equal numbers (regret = weight x (achieved - expected)).  Two correct float32 implementations
that add in a different order therefore agree to about 1e-5 relative on most elements and disagree
freely on the few whose value the arithmetic does not determine: a sum sitting on its threshold, a
quotient of two numbers that are rounding noise, and everything computed from those further down the
tree or up the value backup.

Two comparisons are built on that, both with masks computed from the oracle alone, before the
product is looked at:

* ONE STEP FROM THE SAME STATE (`compare_step`): the oracle is given the product's state tensors,
  both take one iteration, and every entry must agree to 1e-5 relative plus a small absolute part.
  From identical inputs the element-wise arithmetic is identical and only sums over hands are added
  in a different order, so a single cause is left and it is masked explicitly: showdown values (and
  the same player's value of the same hand at the ancestors they are backed up into) whose
  denominator — the opponent mass compatible with the hand, formed as 1 - cs[a] - cs[b] + v in
  float32 (cfr_evaluator.py:577-587) — is below SHOWDOWN_MASS_FLOOR, where the quotient divides
  rounding error by a small number.

* FREE RUNNING (`compare_free`): product and oracle iterate on their own.  Their inputs then differ
  by roundings from the first iteration on, and which entries that leaves undetermined is measured:
  the oracle is run again, several times, from a state in which every entry is multiplied by
  1 + amp * N(0,1) (a few float32 roundings; zeros stay zeros), and an entry is *undetermined* if
  any such twin moves it by more than a third of the tolerance.  Undetermined entries and the
  showdown entries above are exempt, every other entry is held to the tolerance times a stated,
  measured factor per iteration, and the exempt share is bounded per tensor family at twice what the
  suite measures (MAX_EXEMPT), so that the mask cannot swallow a tensor.  Exempt entries are not free
  either: they must be finite and within a coarse tolerance plus a multiple of the twins' own spread.
"""
from __future__ import annotations

import copy

import numpy as np

from oracle import cfr as OCFR
from oracle.unblocked import calculate_unblocked_mass

STATE_NAMES = OCFR.OracleCFR.STATE_NAMES

RTOL = 1e-5
# absolute part of the tolerance, by the natural size of the entries: ranges and reach
# probabilities are <= 1 and mostly ~1e-3, policies are <= 1, values and regrets are chips over
# the starting stack (|v| <= 1, regrets a few units after many iterations)
ATOL = {"policy_probs": 1e-6, "policy_probs_avg": 1e-6, "policy_probs_sample": 1e-6,
        "cumulative_regrets": 2e-6, "regret_weight_sums": 2e-6,
        "self_reach": 1e-6, "self_reach_avg": 1e-6, "beliefs": 1e-7, "beliefs_avg": 1e-7,
        "latest_values": 2e-6, "values_avg": 2e-6}


SHOWDOWN_MASS_FLOOR = 0.05


def showdown_noise(orc, floor: float = SHOWDOWN_MASS_FLOOR) -> np.ndarray:
    """[total, 2, 1326] bool: showdown values whose denominator is below `floor`, and the entries of
    the same player and hand at every ancestor (the value backup works hand by hand)."""
    beliefs = orc.beliefs_avg if orc.cfr_avg else orc.beliefs
    mask = np.zeros(orc.latest_values.shape, dtype=bool)
    sd = np.unique(orc.showdown_indices)
    if sd.size:
        mask[sd] = calculate_unblocked_mass(beliefs[sd][:, ::-1, :]) < np.float32(floor)   # hero p faces range 1 - p
    for d in range(orc.tree_depth - 1, -1, -1):
        s, e = orc.depth_offsets[d + 1], orc.depth_offsets[d + 2]
        np.logical_or.at(mask, orc.parent_index[s:e], mask[s:e])
    return mask


def state_of(ev) -> dict:
    """The evaluator's state tensors as numpy arrays."""
    return {name: getattr(ev, name).detach().cpu().numpy() for name in STATE_NAMES}


def set_state(orc, state: dict, last_model_values=None) -> None:
    for name in STATE_NAMES:
        getattr(orc, name)[...] = state[name]
    if last_model_values is not None:
        orc.last_model_values = np.array(last_model_values, dtype=np.float32)


def _perturb(orc, rng, amp):
    for name in STATE_NAMES:
        arr = getattr(orc, name)
        arr *= (1.0 + amp * rng.standard_normal(arr.shape)).astype(np.float32)
    if getattr(orc, "last_model_values", None) is not None:
        lm = orc.last_model_values
        lm *= (1.0 + amp * rng.standard_normal(lm.shape)).astype(np.float32)


class OracleWithTwins:
    """The oracle plus `n_twins` copies of it that start from inputs one rounding away."""

    def __init__(self, orc, n_twins: int = 3, amp: float = 1e-6, seed: int = 0):
        self.base = orc
        self.amp = amp
        self.rng = np.random.default_rng(seed)
        self.twins = [copy.deepcopy(orc) for _ in range(n_twins)]
        for tw in self.twins:
            _perturb(tw, self.rng, amp)
        # showdown quotients over rounding noise seen at ANY iteration so far: the running average of the
        # values keeps what such a quotient once put into it
        self.noise_history = showdown_noise(orc)

    def set_state(self, state: dict, last_model_values=None) -> None:
        """Teacher forcing: the oracle continues from `state` (name -> array), the twins from that
        state one rounding away."""
        for o in [self.base] + self.twins:
            for name in STATE_NAMES:
                getattr(o, name)[...] = state[name]
            if last_model_values is not None:
                o.last_model_values = np.array(last_model_values, dtype=np.float32)
        for tw in self.twins:
            _perturb(tw, self.rng, self.amp)

    def cfr_iteration(self, t: int) -> None:
        for o in [self.base] + self.twins:
            o.cfr_iteration(t)
        self.noise_history = self.noise_history | showdown_noise(self.base)

    def __getattr__(self, name):           # everything else reads through to the oracle itself
        return getattr(self.base, name)

    def undetermined(self, name: str, rtol: float, atol: float, share: float = 1.0 / 3.0) -> np.ndarray:
        b = getattr(self.base, name)
        tol = share * (atol + rtol * np.abs(b))
        mask = np.zeros(b.shape, dtype=bool)
        for tw in self.twins:
            mask |= np.abs(getattr(tw, name) - b) > tol
        return mask

    def spread(self, name: str) -> np.ndarray:
        """How far the twins move each entry: the oracle's own uncertainty about it."""
        b = getattr(self.base, name)
        out = np.zeros(b.shape, dtype=np.float32)
        for tw in self.twins:
            np.maximum(out, np.abs(getattr(tw, name) - b), out=out)
        return out


# Entries exempt because the arithmetic leaves them open still have to be numbers of the right size:
# finite, and within COARSE_RTOL / COARSE_ATOL of the oracle plus SPREAD_FACTOR times what the oracle's
# own twins move the entry by (an entry that a rounding moves by 0.1 in the oracle cannot be held to
# 3e-4 in the product).  Only quotients over a denominator that is rounding noise (`noise_mask`: the
# showdown entries of SHOWDOWN_MASS_FLOOR, for the running average of the values at any iteration so
# far) may be anything finite.
COARSE_RTOL, COARSE_ATOL, SPREAD_FACTOR = 1e-3, 3e-4, 3.0

# Largest share of a tensor that may be exempt, per kind of comparison and tensor family: twice the
# largest share measured over the whole suite on the MI355X (in brackets; the session report printed by
# tests/conftest.py shows the current figures).  The one-step comparison exempts showdown quotients over
# rounding noise only (largest seen 2.15e-3 of the value entries).
FAMILY = {"policy_probs": "policy", "policy_probs_avg": "policy", "policy_probs_sample": "policy",
          "cumulative_regrets": "regrets", "regret_weight_sums": "regrets", "self_reach": "reach",
          "self_reach_avg": "reach", "beliefs": "beliefs", "beliefs_avg": "beliefs", "latest_values": "values",
          "values_avg": "values"}
STEP_MAX_EXEMPT = 4e-3
MAX_EXEMPT = {
    # product and oracle each iterating on their own, leaves terminal or zero
    "free running": {"policy": 0.24,      # [0.118]
                     "regrets": 0.18,     # [0.091]
                     "reach": 0.30,       # [0.154]
                     "beliefs": 0.03,     # [0.014]
                     "values": 0.05},     # [0.025]
    # the same with a network at the leaves: its answers move with the leaves' ranges, which reach leaves open
    "free running, network at the leaves": {"policy": 0.34,    # [0.168]
                                            "regrets": 0.25,   # [0.125]
                                            "reach": 0.42,     # [0.212]
                                            "beliefs": 0.13,   # [0.067]
                                            "values": 0.43},   # [0.216]
    # the oracle (CPU) and the product against the vectors of the reference's own runs (64 stored columns)
    "oracle against the reference fixtures": {"policy": 0.15,  # [0.072]
                                              "regrets": 0.09,  # [0.042]
                                              "reach": 0.26,    # [0.126]
                                              "beliefs": 0.08,  # [0.038]
                                              "values": 0.04},  # [0.018]
    "reference fixture, fused class": {"policy": 0.15,         # [0.072]
                                       "regrets": 0.09,        # [0.042]
                                       "reach": 0.26,          # [0.128]
                                       "beliefs": 0.04,        # [0.019]
                                       "values": 0.035},       # [0.015]
    # against the base class's vectors the board-blocked hands (a quarter of the stored columns) are
    # exempt by design: the product follows the fused class there
    "reference fixture, base class": {"policy": 0.54,          # [0.270]
                                      "regrets": 0.55,         # [0.276]
                                      "reach": 0.66,           # [0.331]
                                      "beliefs": 0.54,         # [0.270]
                                      "values": 0.50},         # [0.251]
}


def cap_for(kind: str, name: str) -> float:
    return MAX_EXEMPT.get(kind, MAX_EXEMPT["free running"])[FAMILY[name]]


# What the comparisons measured, kept per kind of comparison and tensor for the report that
# tests/conftest.py prints at the end of a session: kind -> name -> {exempt, worst, p999, coarse}.
MEASURED: dict = {}


def _check(what, name, a, e, exempt_mask, rtol, atol, factor, max_exempt, noise_mask=None, kind="other", spread=None):
    err = np.abs(a - e)
    tol = atol + rtol * np.abs(e)
    ratio = np.where(exempt_mask, 0.0, err / tol)
    exempt = float(exempt_mask.mean()) if exempt_mask.size else 0.0
    worst = float(ratio.max()) if ratio.size else 0.0
    assert np.isfinite(a).all(), f"{what}{name}: {int((~np.isfinite(a)).sum())} entries are not finite"
    assert worst <= factor, (
        f"{what}{name}: {int((ratio > factor).sum())} of {ratio.size} entries beyond {factor:g} x tolerance "
        f"(rtol {rtol:g}, atol {atol:g}); worst {worst:.2f} x at index "
        f"{np.unravel_index(int(np.argmax(ratio)), ratio.shape)}; exempt share {exempt:.2e}")
    assert exempt <= max_exempt, f"{what}{name}: {exempt:.2e} of the tensor is exempt (cap {max_exempt:g})"
    open_mask = exempt_mask if noise_mask is None else exempt_mask & ~noise_mask
    coarse_tol = COARSE_ATOL + COARSE_RTOL * np.abs(e) + (SPREAD_FACTOR * spread if spread is not None else 0.0)
    coarse = np.where(open_mask, err / coarse_tol, 0.0)
    worst_coarse = float(coarse.max()) if coarse.size else 0.0
    assert worst_coarse <= 1.0, (
        f"{what}{name}: {int((coarse > 1.0).sum())} exempt entries beyond the coarse bound (rtol {COARSE_RTOL:g}, "
        f"atol {COARSE_ATOL:g}, {SPREAD_FACTOR:g} x the twins' spread); worst {worst_coarse:.2f} x at index "
        f"{np.unravel_index(int(np.argmax(coarse)), coarse.shape)}")
    out = {"worst_over_tol": worst, "p999_over_tol": float(np.quantile(err / tol, 0.999)) if err.size else 0.0,
           "exempt": exempt, "coarse": worst_coarse}
    seen = MEASURED.setdefault(kind, {}).setdefault(name, {"exempt": 0.0, "worst": 0.0, "p999": 0.0, "coarse": 0.0, "n": 0})
    seen["exempt"] = max(seen["exempt"], exempt)
    seen["worst"] = max(seen["worst"], worst)
    seen["p999"] = max(seen["p999"], out["p999_over_tol"])
    seen["coarse"] = max(seen["coarse"], worst_coarse)
    seen["n"] += 1
    return out


def measured_report() -> str:
    """The largest exempt share, worst determined entry, 99.9th percentile over all entries (both in
    tolerances) and worst exempt entry (in coarse tolerances) seen so far, per kind of comparison and tensor."""
    lines = []
    for kind in sorted(MEASURED):
        lines.append(f"{kind}:")
        for name, m in MEASURED[kind].items():
            lines.append(f"  {name:22s} comparisons {m['n']:4d}  exempt share {m['exempt']:.4f}  worst determined "
                         f"{m['worst']:.2f}  p99.9 of all {m['p999']:.2f}  worst exempt (coarse) {m['coarse']:.3f}")
    return "\n".join(lines)


VALUE_TENSORS = ("latest_values", "values_avg")


def compare_step(got: dict, orc, rtol: float = RTOL, names=None, max_exempt: float = STEP_MAX_EXEMPT,
                 what: str = "") -> dict:
    """One iteration from the same state: every entry within rtol * |oracle| + ATOL, except
    showdown quotients with a denominator below SHOWDOWN_MASS_FLOOR and what is backed up from them."""
    noise = showdown_noise(orc)
    report = {}
    for name in names or STATE_NAMES:
        ref = getattr(orc, name)
        mask = noise if name in VALUE_TENSORS else np.zeros(ref.shape, dtype=bool)
        report[name] = _check(what, name, got[name], ref, mask, rtol, ATOL[name], 1.0, max_exempt, noise_mask=mask,
                              kind="one step from the same state")
    return report


def compare_free(got: dict, pack: OracleWithTwins, factor: float = 1.0, rtol: float = RTOL, names=None,
                 max_exempt: float | None = None, expected: dict | None = None, select=None, also_exempt=None,
                 what: str = "", kind: str = "free running") -> dict:
    """Free-running comparison: entries the oracle determines (see the module docstring) within
    `factor` x (rtol * |expected| + ATOL) of `expected` (default: the oracle's own state).
    `select(name, array)` restricts every array, e.g. to the columns a fixture stores;
    `also_exempt(name)` may return a further mask (shape after `select`), e.g. hands on which two
    classes of the reference legitimately differ."""
    noise = showdown_noise(pack.base)
    report = {}
    for name in names or STATE_NAMES:
        ref = getattr(pack.base, name)
        mask = pack.undetermined(name, rtol, ATOL[name])
        spread = pack.spread(name)
        if name == "values_avg":
            loose = noise | getattr(pack, "noise_history", noise)
        else:
            loose = noise if name in VALUE_TENSORS else np.zeros(ref.shape, dtype=bool)
        mask = mask | loose
        a = got[name]
        e = ref if expected is None else expected[name]
        if select is not None:
            mask = select(name, mask)
            loose = select(name, loose)
            spread = select(name, spread)
            a = a if a.shape == mask.shape else select(name, a)
            e = e if e.shape == mask.shape else select(name, e)
        if also_exempt is not None:
            extra = also_exempt(name)
            if extra is not None:
                mask = mask | np.broadcast_to(extra, mask.shape)
                loose = loose | np.broadcast_to(extra, mask.shape)
        cap = cap_for(kind, name) if max_exempt is None else max_exempt
        report[name] = _check(what, name, a, e, mask, rtol, ATOL[name], factor, cap, noise_mask=loose, kind=kind,
                              spread=spread)
    return report


def worst_of(report: dict) -> float:
    return max(r["worst_over_tol"] for r in report.values())
