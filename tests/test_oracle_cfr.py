"""CPU: pins the oracle's CFR restatement with things the reference cannot supply here
(its evaluator is not importable: hydra / omegaconf are absent):

  * structural identities after every iteration;
  * the base and the fused variants of the restatement agree wherever probability mass lives;
  * an INDEPENDENT textbook CFR / best-response on the explicit two-player game (a handful of
    live combos per player, every compatible hand pair enumerated) agrees with the oracle on
    the game value, and finds the oracle's average strategy nearly unexploitable.
"""
import numpy as np
import pytest

from oracle import cards as OC
from oracle import cfr as OCFR
from oracle import tree as OT
from oracle.ranker import rank_hands
from tests.helpers import C, random_boards, random_ranges


def river_tree(n_roots, depth=2, pot=200, stack=800):
    roots = [OT.make_root(3, pot, stack, stack, button=i % 2) for i in range(n_roots)]
    return OT.build_tree(roots, [0.5, 1.0], depth)


def test_structural_identities_every_iteration():
    rng = np.random.default_rng(4)
    n = 2
    t = river_tree(n)
    boards = random_boards(rng, n)
    bel = random_ranges(rng, boards)
    o = OCFR.OracleCFR(t, boards, bel, cfr_iterations=12, enforce_zero_sum=True)
    o.prepare()
    top = o.depth_offsets[-2]
    parents = np.nonzero(o.child_count[:top] > 0)[0]
    for it in range(12):
        o.cfr_iteration(it)
        for pol in (o.policy_probs, o.policy_probs_avg):
            s = np.zeros((top, 1326), np.float32)
            o.pull_back_sum(pol, s)
            np.testing.assert_allclose(s[parents], 1.0, atol=2e-6)
        for b in (o.beliefs, o.beliefs_avg):
            np.testing.assert_allclose(b.sum(-1), 1.0, atol=2e-6)
            assert (b[np.broadcast_to(~o.allowed_hands[:, None, :], b.shape)] == 0).all()
        par = o.parent_index[n:]
        assert (o.self_reach[n:] <= o.self_reach[par] + 1e-7).all()
        # zero-sum step: sum_p sum_h v_p b_p = 0 on non-terminal rows
        zs = (o.values_avg * o.beliefs_avg).sum(-1).sum(-1)
        assert np.abs(zs[~o.done]).max() < 2e-6
        assert np.isfinite(o.values_avg).all() and np.abs(o.latest_values).max() <= 1.0 + 1e-5


def test_base_and_fused_variants_agree_on_live_hands():
    rng = np.random.default_rng(5)
    n = 2
    t = river_tree(n)
    boards = random_boards(rng, n)
    bel = random_ranges(rng, boards)
    a = OCFR.OracleCFR(t, boards, bel, cfr_iterations=15, dcfr_delay=3)
    b = OCFR.OracleCFR(t, boards, bel, cfr_iterations=15, dcfr_delay=3, fused_variant=True)
    a.prepare(); b.prepare()
    for it in range(15):
        a.cfr_iteration(it); b.cfr_iteration(it)
    for name in OCFR.OracleCFR.STATE_NAMES:
        x, y = getattr(a, name), getattr(b, name)
        m = a.allowed_hands if x.ndim == 2 else np.broadcast_to(a.allowed_hands[:, None, :], x.shape)
        np.testing.assert_allclose(x[m], y[m], rtol=1e-3, atol=1e-4, err_msg=name)  # roundings differ, nothing else


# ---------------------------------------------------------------------------------------
# Independent textbook solver on the explicit game (no code shared with oracle/cfr.py).
class TinyGame:
    """River subgame with a few live combos per player.  Pure-python recursion over the tree
    dict; a strategy is sigma[node][hand_index] -> probabilities over that node's children."""

    def __init__(self, tree, board, hands0, hands1, prior0, prior1):
        self.t = tree
        self.h = (list(hands0), list(hands1))
        self.prior = (np.asarray(prior0, float), np.asarray(prior1, float))
        cm = OC.hand_combos()
        ranks = rank_hands(np.asarray(board)[None])[0][0]
        k0, k1 = len(hands0), len(hands1)
        self.compat = np.zeros((k0, k1))
        self.sign = np.zeros((k0, k1))
        for i, a in enumerate(hands0):
            for j, b in enumerate(hands1):
                if len(set(cm[a]) | set(cm[b])) == 4:
                    self.compat[i, j] = 1.0
                    self.sign[i, j] = np.sign(int(ranks[a]) - int(ranks[b]))
        self.joint = self.prior[0][:, None] * self.prior[1][None, :] * self.compat
        self.joint /= self.joint.sum()
        self.children = {}
        for p in range(tree["depth_offsets"][-1]):
            cnt = int(tree["child_count"][p])
            self.children[p] = list(range(int(tree["child_offsets"][p]), int(tree["child_offsets"][p]) + cnt)) if cnt else []

    def terminal_u0(self, node):
        """Utility of player 0 per hand pair at a leaf, in units of `scale`."""
        t = self.t
        if t["fold_mask"][node]:
            return np.full_like(self.compat, float(t["reward"][node]))
        if t["showdown_mask"][node]:
            pot = t["showdown_potential"][node] / float(t["scale"][node])
            assert pot[0] == pot[1]
            return self.sign * pot[0]
        return np.zeros_like(self.compat)  # depth-limited leaf: value 0 (zero leaf model)

    def uniform(self):
        return {p: [np.full(len(ch), 1.0 / len(ch)) for _ in self.h[int(self.t["to_act"][p])]]
                for p, ch in self.children.items() if ch}

    def value(self, sigma, node=0):
        """u0[h0,h1] of the profile below `node`."""
        ch = self.children[node]
        if not ch:
            return self.terminal_u0(node)
        actor = int(self.t["to_act"][node])
        out = np.zeros_like(self.compat)
        for k, c in enumerate(ch):
            u = self.value(sigma, c)
            w = np.array([sigma[node][i][k] for i in range(len(self.h[actor]))])
            out += u * (w[:, None] if actor == 0 else w[None, :])
        return out

    def game_value(self, sigma):
        return float((self.joint * self.value(sigma)).sum())

    def best_response_value(self, sigma, br_player):
        """Value (for br_player) of the best response against sigma's other player."""
        def rec(node, reach_opp):
            # returns per-hand counterfactual value vector of br_player: sum over opp hands
            ch = self.children[node]
            if not ch:
                u0 = self.terminal_u0(node)
                u = u0 if br_player == 0 else -u0
                jw = self.joint * (reach_opp[None, :] if br_player == 0 else reach_opp[:, None])
                return (jw * u).sum(axis=1 - br_player if br_player == 0 else 0)
            actor = int(self.t["to_act"][node])
            if actor == br_player:
                vals = np.stack([rec(c, reach_opp) for c in ch])
                return vals.max(axis=0)
            tot = 0.0
            for k, c in enumerate(ch):
                w = np.array([sigma[node][i][k] for i in range(len(self.h[actor]))])
                tot = tot + rec(c, reach_opp * w)
            return tot
        return float(rec(0, np.ones(len(self.h[1 - br_player]))).sum())

    def exploitability(self, sigma):
        return 0.5 * (self.best_response_value(sigma, 0) + self.best_response_value(sigma, 1))

    def node_tables(self, sigma):
        """Per node, under strategy sigma: each player's expected value per own hand GIVEN that
        the hand is held there (opponent hands weighted by prior x opponent reach x compatibility),
        and the actor's per-action regrets weighted by the opponent's normalised beliefs."""
        out = {}

        def rec(node, r0, r1):
            ch = self.children[node]
            us = None
            if not ch:
                u = self.terminal_u0(node)
            else:
                actor = int(self.t["to_act"][node])
                w = [np.array([sigma[node][i][k] for i in range(len(self.h[actor]))]) for k in range(len(ch))]
                us = [rec(c, r0 * w[k] if actor == 0 else r0, r1 * w[k] if actor == 1 else r1)
                      for k, c in enumerate(ch)]
                u = sum(us[k] * (w[k][:, None] if actor == 0 else w[k][None, :]) for k in range(len(ch)))
            w0, w1 = self.prior[0] * r0, self.prior[1] * r1
            b0, b1 = w0 / w0.sum(), w1 / w1.sum()
            m0 = (self.compat * b1[None, :]).sum(axis=1)
            m1 = (self.compat * b0[:, None]).sum(axis=0)
            entry = {"v0": (self.compat * b1[None, :] * u).sum(axis=1) / np.maximum(m0, 1e-300),
                     "v1": (self.compat * b0[:, None] * -u).sum(axis=0) / np.maximum(m1, 1e-300),
                     "m0": m0, "m1": m1, "r0": r0.copy(), "r1": r1.copy()}
            if ch:
                if actor == 0:
                    entry["regret"] = [(self.compat * b1[None, :] * (uk - u)).sum(axis=1) for uk in us]
                else:
                    entry["regret"] = [(self.compat * b0[:, None] * -(uk - u)).sum(axis=0) for uk in us]
            out[node] = entry
            return u

        rec(0, np.ones(len(self.h[0])), np.ones(len(self.h[1])))
        return out

    def solve(self, iters, belief_normalised=False, on_iteration=None):
        """Vanilla CFR with simultaneous updates; returns the average strategy.

        belief_normalised=True divides every counterfactual regret by the opponent's total
        probability of reaching the node, which is what regrets computed from per-node
        NORMALISED beliefs amount to (the reference's choice, cfr_evaluator.py:1244-1262).
        on_iteration(k, sigma, min_z) sees the strategy after k regret updates."""
        regret = {p: [np.zeros(len(ch)) for _ in self.h[int(self.t["to_act"][p])]]
                  for p, ch in self.children.items() if ch}
        strat_sum = {p: [np.zeros(len(ch)) for _ in self.h[int(self.t["to_act"][p])]]
                     for p, ch in self.children.items() if ch}

        def sigma_now():
            out = {}
            for p, rs in regret.items():
                out[p] = []
                for r in rs:
                    pos = np.maximum(r, 0)
                    out[p].append(pos / pos.sum() if pos.sum() > 0 else np.full(len(r), 1.0 / len(r)))
            return out

        def rec(node, sig, r0, r1):
            ch = self.children[node]
            if not ch:
                return self.terminal_u0(node)
            actor = int(self.t["to_act"][node])
            us = [rec(c, sig,
                      r0 * np.array([sig[node][i][k] for i in range(len(self.h[0]))]) if actor == 0 else r0,
                      r1 * np.array([sig[node][i][k] for i in range(len(self.h[1]))]) if actor == 1 else r1)
                  for k, c in enumerate(ch)]
            w = [np.array([sig[node][i][k] for i in range(len(self.h[actor]))]) for k in range(len(ch))]
            u = sum(us[k] * (w[k][:, None] if actor == 0 else w[k][None, :]) for k in range(len(ch)))
            if actor == 0:
                z = float((self.prior[1] * r1).sum())
                cf = [(self.joint * r1[None, :] * us[k]).sum(axis=1) for k in range(len(ch))]
                cfn = (self.joint * r1[None, :] * u).sum(axis=1)
                reach_self = r0
            else:
                z = float((self.prior[0] * r0).sum())
                cf = [(self.joint * r0[:, None] * -us[k]).sum(axis=0) for k in range(len(ch))]
                cfn = (self.joint * r0[:, None] * -u).sum(axis=0)
                reach_self = r1
            min_z[0] = min(min_z[0], z)
            scale = 1.0 / max(z, 1e-30) if belief_normalised else 1.0
            for i in range(len(self.h[actor])):
                for k in range(len(ch)):
                    regret[node][i][k] += (cf[k][i] - cfn[i]) * scale
                    strat_sum[node][i][k] += reach_self[i] * sig[node][i][k]
            return u

        min_z = [1.0]
        for k in range(iters):
            rec(0, sigma_now(), np.ones(len(self.h[0])), np.ones(len(self.h[1])))
            if on_iteration is not None:
                on_iteration(k + 1, sigma_now(), min_z[0])
        avg = {}
        for p, ss in strat_sum.items():
            avg[p] = [s / s.sum() if s.sum() > 0 else np.full(len(s), 1.0 / len(s)) for s in ss]
        return avg


def tiny_setup(depth):
    board = np.array([C(12, 0), C(9, 1), C(5, 3), C(3, 0), C(0, 2)])   # As Jh 7c 5s 2d
    combo = OC.combo_index
    hands0 = [combo(C(12, 1), C(11, 1)), combo(C(9, 0), C(9, 2)), combo(C(10, 3), C(8, 3)), combo(C(5, 0), C(4, 0)),
              combo(C(11, 2), C(10, 2))]
    hands1 = [combo(C(12, 2), C(3, 3)), combo(C(9, 3), C(8, 1)), combo(C(6, 1), C(6, 2)), combo(C(11, 0), C(2, 1)),
              combo(C(12, 1), C(7, 1))]   # the last one shares the ace of hearts with hands0[0]
    p0 = np.array([0.3, 0.2, 0.2, 0.2, 0.1])
    p1 = np.array([0.15, 0.25, 0.2, 0.25, 0.15])
    t = OT.build_tree([OT.make_root(3, 200, 800, 800, button=0)], [0.5, 1.0], depth)
    bel = np.zeros((1, 2, 1326), np.float32)
    bel[0, 0, hands0] = p0
    bel[0, 1, hands1] = p1
    return board, hands0, hands1, p0, p1, t, bel


def oracle_strategy(game, t, policy):
    """A [total, 1326] policy tensor restricted to the explicit game's live hands."""
    sig = {}
    for p, ch in game.children.items():
        if not ch:
            continue
        rows = []
        for h in game.h[int(t["to_act"][p])]:
            v = np.array([policy[c, h] for c in ch], dtype=float)
            rows.append(v / v.sum() if v.sum() > 0 else np.full(len(ch), 1.0 / len(ch)))
        sig[p] = rows
    return sig


def random_policy(rng, game, t, total):
    """A strictly positive random strategy: explicit-game form and [total, 1326] tensor form."""
    policy = np.zeros((total, 1326), np.float32)
    sigma = {}
    for p, ch in game.children.items():
        if not ch:
            continue
        x = rng.dirichlet(np.ones(len(ch)) * 1.5, size=1326).T.astype(np.float32)   # [children, 1326]
        x = np.maximum(x, np.float32(0.02))
        x /= x.sum(axis=0, keepdims=True)
        policy[ch] = x
        sigma[p] = [np.array([float(policy[c, h]) for c in ch]) for h in game.h[int(t["to_act"][p])]]
        for row in sigma[p]:
            row /= row.sum()
    return sigma, policy


@pytest.mark.parametrize("depth", [2, 3, 4])
def test_oracle_values_and_regrets_match_explicit_game(depth):
    """For a random full-support strategy, one pass of reach -> beliefs -> leaf values -> backup ->
    regrets in the oracle equals the same quantities computed pair by pair on the explicit game.
    Pins the level-major plumbing, the opponent-conditioned backup, blockers, fold / showdown
    values and the regret weights at every depth, in a representation that shares nothing with
    the oracle (no 1326-vectors, no prefix sums, no inclusion-exclusion)."""
    board, hands0, hands1, p0, p1, t, bel = tiny_setup(depth)
    game = TinyGame(t, board, hands0, hands1, p0, p1)
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=4)
    o.prepare()
    rng = np.random.default_rng(100 + depth)
    sigma, policy = random_policy(rng, game, t, o.total_nodes)
    o.policy_probs[:] = policy
    o.calculate_reach_weights(o.self_reach, o.policy_probs)
    o.propagate_all_beliefs(o.beliefs, o.self_reach)
    o.set_leaf_values(0)
    o.compute_expected_values()
    regrets = o.compute_instantaneous_regrets(o.latest_values)
    tab = game.node_tables(sigma)
    hs = (np.array(hands0), np.array(hands1))
    for node, e in tab.items():
        np.testing.assert_allclose(o.self_reach[node, 0, hs[0]], e["r0"], rtol=2e-5, atol=1e-7, err_msg=f"reach {node}")
        np.testing.assert_allclose(o.self_reach[node, 1, hs[1]], e["r1"], rtol=2e-5, atol=1e-7, err_msg=f"reach {node}")
        live0, live1 = e["m0"] > 0, e["m1"] > 0
        np.testing.assert_allclose(o.latest_values[node, 0, hs[0]][live0], e["v0"][live0], atol=2e-6, rtol=2e-5,
                                   err_msg=f"values p0 node {node}")
        np.testing.assert_allclose(o.latest_values[node, 1, hs[1]][live1], e["v1"][live1], atol=2e-6, rtol=2e-5,
                                   err_msg=f"values p1 node {node}")
        if "regret" in e:
            actor = int(t["to_act"][node])
            for k, c in enumerate(game.children[node]):
                np.testing.assert_allclose(regrets[c, hs[actor]], e["regret"][k], atol=2e-6, rtol=2e-5,
                                           err_msg=f"regret node {node} child {c}")


@pytest.mark.parametrize("cfr_type,gamma", [("discounted", 2.0), ("standard", None), ("linear", None)])
def test_oracle_average_policy_is_the_reach_weighted_average(cfr_type, gamma):
    """The recursive mix with the reach under the running average (cfr_evaluator.py:1264-1328)
    must equal the closed form  sum_t w_t r_t sigma_t / sum_t w_t r_t  with r_t the actor's own
    reach of the node under sigma_t: the average of realisation plans.  The weights w_t follow
    from the (old, new) pair of each step: w_t = W_{t-1} * new / old."""
    depth = 3
    board, hands0, hands1, p0, p1, t, bel = tiny_setup(depth)
    game = TinyGame(t, board, hands0, hands1, p0, p1)
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=8, cfr_type=cfr_type)
    o.prepare()
    rng = np.random.default_rng(17)
    steps = 6
    hs = (np.array(hands0), np.array(hands1))
    num = {p: np.zeros((len(ch), 5)) for p, ch in game.children.items() if ch}
    den = {p: np.zeros(5) for p in num}
    w_total = 0.0
    for step in range(steps):
        sigma, policy = random_policy(rng, game, t, o.total_nodes)
        o.apply_schedules(step)
        o.policy_probs[:] = policy
        o.calculate_reach_weights(o.self_reach, o.policy_probs)
        o.update_average_policy(step)
        o.calculate_reach_weights(o.self_reach_avg, o.policy_probs_avg)
        if step == 0:
            w = 1.0
        else:
            old, new = o.mixing_weights(step)
            w = w_total * float(new) / float(old)
        w_total += w
        tab = game.node_tables(sigma)
        for p in num:
            actor = int(t["to_act"][p])
            r = tab[p]["r0"] if actor == 0 else tab[p]["r1"]
            den[p] += w * r
            for k in range(len(game.children[p])):
                num[p][k] += w * r * np.array([sigma[p][i][k] for i in range(5)])
    for p, ch in game.children.items():
        if not ch:
            continue
        actor = int(t["to_act"][p])
        np.testing.assert_allclose(o.policy_probs_avg[np.array(ch)][:, hs[actor]], num[p] / den[p][None, :],
                                   rtol=2e-4, atol=2e-6, err_msg=f"node {p}")


@pytest.mark.parametrize("depth", [2])
def test_oracle_policy_trajectory_matches_explicit_game(depth):
    """Iteration by iteration, the oracle's current policy (cfr_type standard: plain regret sums)
    equals regret matching on the explicit hand-pair game with belief-normalised regrets.
    Checks the level-major tree plumbing, reach, the opponent-conditioned backup, blockers and
    showdown/fold values at every depth, in a representation that shares nothing with the oracle.
    The comparison stops when some node's opponent reach falls under 1e-4: below 1e-5 the
    reference replaces the beliefs by a uniform fallback, which the explicit game has no use for."""
    board, hands0, hands1, p0, p1, t, bel = tiny_setup(depth)
    game = TinyGame(t, board, hands0, hands1, p0, p1)
    iters = 30
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=iters, cfr_type="standard")
    o.prepare()
    trace = {}
    game.solve(iters, belief_normalised=True, on_iteration=lambda k, sig, z: trace.__setitem__(k, (sig, z)))
    compared = 0
    for k in range(1, iters + 1):
        o.cfr_iteration(k - 1)
        sig, z = trace[k]
        if z < 1e-4:
            break
        got = oracle_strategy(game, t, o.policy_probs)
        for p in sig:
            np.testing.assert_allclose(np.array(got[p]), np.array(sig[p]), atol=2e-3, err_msg=f"iter {k} node {p}")
        compared += 1
    assert compared >= 5, compared


@pytest.mark.parametrize("depth", [2, 3])
def test_oracle_matches_independent_solver_on_tiny_ranges(depth):
    board, hands0, hands1, p0, p1, t, bel = tiny_setup(depth)
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=400, dcfr_delay=0)
    o.evaluate_cfr()
    game = TinyGame(t, board, hands0, hands1, p0, p1)
    avg = game.solve(1500)
    expl_ref = game.exploitability(avg)
    nash_value = game.game_value(avg)
    assert expl_ref < 2e-3, expl_ref   # the independent solver itself converged (pot = 0.2 units)

    # The oracle's average strategy in the explicit game.  With one decision per player (depth 2)
    # it is nearly unexploitable.  Deeper, the reference's belief-normalised regrets weigh an
    # iteration by 1 / (opponent's reach of the node), which is no longer regret-bounded CFR: the
    # explicit game run with the same weighting hovers between 0.01 and 0.025 (5-12 % of the pot)
    # for thousands of iterations, and so does the oracle; the bound below is that band.
    sig = oracle_strategy(game, t, o.policy_probs_avg)
    expl = game.exploitability(sig)
    tol = 3e-3 if depth == 2 else 5e-2
    assert expl < tol, expl
    assert abs(game.game_value(sig) - nash_value) < tol

    # the oracle's root values weigh back to the same game value
    from oracle.unblocked import calculate_unblocked_mass
    m1 = calculate_unblocked_mass(bel[0, 1])[hands0]      # compatible villain mass per hero hand
    v0 = o.values_avg[0, 0, hands0]
    value_oracle = float((p0 * m1 * v0).sum() / (p0 * m1).sum())
    assert abs(value_oracle - nash_value) < 3e-3


# ---------------------------------------------------------------------------------------
# warm start (cfr_evaluator.py:888-955)
def test_warm_start_model_replays_the_initial_policy_and_model_br_reduces_exploitability():
    from oracle import best_response as OBR
    rng = np.random.default_rng(9)
    n = 2
    t = river_tree(n, depth=3)
    boards = random_boards(rng, n)
    bel = random_ranges(rng, boards)
    logits = rng.standard_normal((t["depth_offsets"][-1], 1326, t["legal_mask"].shape[1])).astype(np.float32)

    def policy_logits(beliefs, rows):
        return logits[rows]
    base = OCFR.OracleCFR(t, boards, bel, cfr_iterations=30, policy_logits_fn=policy_logits)
    base.prepare()
    # `model`: cumulative regrets = policy x weight, so regret matching gives the policy back
    # wherever the action's mean positive regret is > 0, and the weight sums hold the weights
    o = OCFR.OracleCFR(t, boards, bel, cfr_iterations=30, policy_logits_fn=policy_logits,
                       warm_start_iterations=5, warm_start_type="model", warm_start_multiplier=10.0)
    o.initialize_policy_and_beliefs()
    before = o.policy_probs.copy()
    o.warm_start()
    nroot = o.root_nodes
    w = o.regret_weight_sums[nroot:, 0]
    assert (w >= 0).all() and (w > 0).any()
    np.testing.assert_allclose(o.cumulative_regrets[nroot:], before[nroot:] * w[:, None], rtol=1e-6)
    wsum = np.zeros(o.depth_offsets[-2], np.float32)
    np.add.at(wsum, o.parent_index[nroot:] , w)
    full = np.repeat(wsum > 0, o.child_count[: o.depth_offsets[-2]])       # families with some weight
    expect = before[nroot:] * w[:, None]
    fam = np.zeros((o.depth_offsets[-2], 1326), np.float32)
    np.add.at(fam, o.parent_index[nroot:], expect)
    expect = expect / np.maximum(np.repeat(fam, o.child_count[: o.depth_offsets[-2]], axis=0), 1e-30)
    live = full[:, None] & (np.repeat(fam, o.child_count[: o.depth_offsets[-2]], axis=0) > 1e-8)
    np.testing.assert_allclose(o.policy_probs[nroot:][live], expect[live], rtol=1e-5, atol=1e-7)
    # `model_br`: regrets against best-response values push the policy towards the best response
    e0, _ = OBR.compute_exploitability(base)
    b = OCFR.OracleCFR(t, boards, bel, cfr_iterations=30, policy_logits_fn=policy_logits,
                       warm_start_iterations=5, warm_start_type="model_br")
    b.prepare()
    assert (b.regret_weight_sums[nroot:] == np.float32(5.0)).all()
    assert np.abs(b.policy_probs - base.policy_probs).max() > 0.05
    for it in range(5, 30):
        b.cfr_iteration(it)
    e1, _ = OBR.compute_exploitability(b)
    assert (e1 < e0).all()
