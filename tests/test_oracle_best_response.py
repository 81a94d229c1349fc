"""CPU: pins the oracle's best response (src/p2/search/cfr_evaluator.py:603-764) with an exact
best response on the explicit hand-pair game."""
import numpy as np
import pytest

from oracle import best_response as OBR
from oracle import cfr as OCFR
from tests.test_oracle_cfr import TinyGame, random_policy, tiny_setup


def per_hand_best_response(game, sigma, br_player):
    """Exact: the best-responding player's value per own hand at the root, GIVEN the hand
    (opponent hands weighted by prior x compatibility), against sigma of the other player."""
    k = len(game.h[br_player])

    def rec(node, reach_opp):
        # returns, per own hand, sum over opponent hands of prior x reach x compat x utility
        ch = game.children[node]
        if not ch:
            u = game.terminal_u0(node) * game.compat
            if br_player == 0:
                return (u * (game.prior[1] * reach_opp)[None, :]).sum(axis=1)
            return (-u * (game.prior[0] * reach_opp)[:, None]).sum(axis=0)
        actor = int(game.t["to_act"][node])
        if actor == br_player:
            return np.max(np.stack([rec(c, reach_opp) for c in ch]), axis=0)
        total = np.zeros(k)
        for j, c in enumerate(ch):
            w = np.array([sigma[node][i][j] for i in range(len(game.h[actor]))])
            total += rec(c, reach_opp * w)
        return total
    num = rec(0, np.ones(len(game.h[1 - br_player])))
    opp_prior = game.prior[1 - br_player]
    mass = (game.compat * opp_prior[None, :]).sum(axis=1) if br_player == 0 else (game.compat * opp_prior[:, None]).sum(axis=0)
    return num / mass


@pytest.mark.parametrize("depth", [2, 3, 4])
def test_best_response_values_match_exact_best_response(depth):
    board, hands0, hands1, p0, p1, t, bel = tiny_setup(depth)
    game = TinyGame(t, board, hands0, hands1, p0, p1)
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=4)
    o.prepare()
    rng = np.random.default_rng(40 + depth)
    sigma, policy = random_policy(rng, game, t, o.total_nodes)
    o.policy_probs[:] = policy
    o.calculate_reach_weights(o.self_reach, o.policy_probs)
    o.propagate_all_beliefs(o.beliefs, o.self_reach)
    o.set_leaf_values(0)
    o.compute_expected_values()
    on_policy = o.latest_values.copy()
    hs = (np.array(hands0), np.array(hands1))
    for player in (0, 1):
        dev = np.full(o.total_nodes, player, dtype=o.to_act.dtype)
        br = OBR.best_response_values(o, o.policy_probs, o.beliefs, o.latest_values, dev)
        exact = per_hand_best_response(game, sigma, player)
        np.testing.assert_allclose(br[0, player, hs[player]], exact, rtol=2e-5, atol=2e-6)
        assert (br[0, player, hs[player]] >= on_policy[0, player, hs[player]] - 1e-6).all()
        assert (br[0, player, hs[player]] > on_policy[0, player, hs[player]] + 1e-4).any()   # random play is exploitable


def test_exploitability_of_a_solved_game_is_small_and_of_uniform_play_large():
    board, _, _, _, _, t, bel = tiny_setup(2)
    o = OCFR.OracleCFR(t, board[None], bel, cfr_iterations=300, use_final_policy_values=False)
    o.prepare()
    expl0, _ = OBR.compute_exploitability(o)          # uniform average policy
    for it in range(300):
        o.cfr_iteration(it)
    expl, br = OBR.compute_exploitability(o)
    assert expl0[0] > 0.02 and expl[0] < expl0[0] / 5
    assert br.shape == (1, 2)
