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
  measured factor per iteration, and the exempt share is bounded so that the mask cannot swallow
  a tensor.
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

    def __getattr__(self, name):           # everything else reads through to the oracle itself
        return getattr(self.base, name)

    def undetermined(self, name: str, rtol: float, atol: float, share: float = 1.0 / 3.0) -> np.ndarray:
        b = getattr(self.base, name)
        tol = share * (atol + rtol * np.abs(b))
        mask = np.zeros(b.shape, dtype=bool)
        for tw in self.twins:
            mask |= np.abs(getattr(tw, name) - b) > tol
        return mask


def _check(what, name, a, e, exempt_mask, rtol, atol, factor, max_exempt):
    err = np.abs(a - e)
    tol = atol + rtol * np.abs(e)
    ratio = np.where(exempt_mask, 0.0, err / tol)
    exempt = float(exempt_mask.mean()) if exempt_mask.size else 0.0
    worst = float(ratio.max()) if ratio.size else 0.0
    assert worst <= factor, (
        f"{what}{name}: {int((ratio > factor).sum())} of {ratio.size} entries beyond {factor:g} x tolerance "
        f"(rtol {rtol:g}, atol {atol:g}); worst {worst:.2f} x at index "
        f"{np.unravel_index(int(np.argmax(ratio)), ratio.shape)}; exempt share {exempt:.2e}")
    assert exempt <= max_exempt, f"{what}{name}: {exempt:.2e} of the tensor is exempt (cap {max_exempt:g})"
    return {"worst_over_tol": worst, "p999_over_tol": float(np.quantile(err / tol, 0.999)) if err.size else 0.0,
            "exempt": exempt}


VALUE_TENSORS = ("latest_values", "values_avg")


def compare_step(got: dict, orc, rtol: float = RTOL, names=None, max_exempt: float = 2e-3, what: str = "") -> dict:
    """One iteration from the same state: every entry within rtol * |oracle| + ATOL, except
    showdown quotients with a denominator below SHOWDOWN_MASS_FLOOR and what is backed up from them."""
    noise = showdown_noise(orc)
    report = {}
    for name in names or STATE_NAMES:
        ref = getattr(orc, name)
        mask = noise if name in VALUE_TENSORS else np.zeros(ref.shape, dtype=bool)
        report[name] = _check(what, name, got[name], ref, mask, rtol, ATOL[name], 1.0, max_exempt)
    return report


def compare_free(got: dict, pack: OracleWithTwins, factor: float = 1.0, rtol: float = RTOL, names=None,
                 max_exempt: float = 0.25, expected: dict | None = None, select=None, also_exempt=None,
                 what: str = "") -> dict:
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
        if name in VALUE_TENSORS:
            mask = mask | noise
        a = got[name]
        e = ref if expected is None else expected[name]
        if select is not None:
            mask = select(name, mask)
            a = a if a.shape == mask.shape else select(name, a)
            e = e if e.shape == mask.shape else select(name, e)
        if also_exempt is not None:
            extra = also_exempt(name)
            if extra is not None:
                mask = mask | np.broadcast_to(extra, mask.shape)
        report[name] = _check(what, name, a, e, mask, rtol, ATOL[name], factor, max_exempt)
    return report


def worst_of(report: dict) -> float:
    return max(r["worst_over_tol"] for r in report.values())
