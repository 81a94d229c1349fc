"""Leaf value networks for the evaluator and the chance node in front of them.

The evaluator asks its ``model`` for ``leaf_values(beliefs[K,2,1326], node_rows[K], evaluator)``.
``ChanceLeafModel`` answers with a PyTorch network: leaves in the middle of a betting round
are evaluated on their own board; leaves where the round has ended and a card is still to
come are expanded over every card that can come next (blocker masking, renormalisation,
network, mean — the semantics of ``ChanceNodeHelper.single_card_chance_values``,
src/p2/search/chance_node_helper.py:360-479), and leaves where the preflop round has ended
over the canonical flops (``flop_chance_values``, :219-357).  The network stays ordinary PyTorch; only the
expansion and the mean are HIP kernels.

``RangeBoardMLP`` is the network of the turn benchmark configuration: input 2 x 1326 ranges +
52-dim board one-hot, three hidden ReLU layers, output 2 x 1326; orthogonal initialisation with
zero biases as in src/p2/models/mlp/rebel_ffn.py:139-148.
"""
from __future__ import annotations

from types import SimpleNamespace

import numpy as np
import torch

from .card_utils import NUM_HANDS
from .chance_node_helper import ChanceNodeHelper, MLPFeatures


class RangeBoardMLP(torch.nn.Module):
    def __init__(self, hidden: int = 1536, layers: int = 3, seed: int = 42) -> None:
        super().__init__()
        dims = [2 * NUM_HANDS + 52] + [hidden] * layers + [2 * NUM_HANDS]
        self.linears = torch.nn.ModuleList(torch.nn.Linear(a, b) for a, b in zip(dims[:-1], dims[1:]))
        gen = torch.Generator().manual_seed(seed)
        for lin in self.linears:
            torch.nn.init.orthogonal_(lin.weight, generator=gen)
            torch.nn.init.zeros_(lin.bias)

    def forward(self, features: MLPFeatures) -> SimpleNamespace:
        board = features.board
        onehot = torch.zeros(board.shape[0], 53, dtype=features.beliefs.dtype, device=board.device)
        onehot.scatter_(1, torch.where(board >= 0, board, torch.full_like(board, 52)), 1.0)
        x = torch.cat([features.beliefs, onehot[:, :52]], dim=1)
        return self.forward_input(x)

    # The input matrix is [ranges (2 x 1326) | board one-hot (52)].  Only the ranges change between the
    # iterations of a search, so a caller may keep the matrix, have the ranges written into its first
    # 2652 columns (HipSparseCFREvaluator.gather_leaf_rows does that in the matrix's dtype) and call
    # forward_input: no concatenation and no separate cast per call.
    input_width = 2 * NUM_HANDS + 52
    # context, street and player to act are not read: a caller that can produce [ranges | board one-hot]
    # rows itself (the chance-node expansion does) may skip the feature bundle altogether
    input_layout = "ranges|board_onehot"

    def static_input_columns(self, features: MLPFeatures, dtype: torch.dtype) -> torch.Tensor:
        """[N, input_width] with the columns that do not depend on the ranges filled in."""
        board = features.board
        onehot = torch.zeros(board.shape[0], 53, dtype=dtype, device=board.device)
        onehot.scatter_(1, torch.where(board >= 0, board, torch.full_like(board, 52)), 1.0)
        x = torch.zeros(board.shape[0], self.input_width, dtype=dtype, device=board.device)
        x[:, 2 * NUM_HANDS:] = onehot[:, :52]
        return x

    def forward_input(self, x: torch.Tensor) -> SimpleNamespace:
        for lin in self.linears[:-1]:
            x = torch.relu(lin(x))
        x = self.linears[-1](x)
        return SimpleNamespace(hand_values=x.view(-1, 2, NUM_HANDS))


def _accepts_keyword(fn, name: str) -> bool:
    """Whether ``fn`` can be called with the keyword ``name``."""
    import inspect
    try:
        params = inspect.signature(fn).parameters.values()
    except (TypeError, ValueError):
        return False
    return any(p.name == name or p.kind is inspect.Parameter.VAR_KEYWORD for p in params)


class NetworkLeafModel:
    """The reference's own leaf rule (src/p2/search/cfr_evaluator.py:1024-1040): the network sees
    the encoded features of every leaf that is not terminal; a leaf that closed a betting round
    is encoded with the board before the next deal, so the network itself stands for the chance
    node.  The initial policy comes from the same network's ``policy_logits`` (:305-329), uniform over
    the legal actions if it has none.  ``HipSparseCFREvaluator`` wraps a bare network — anything
    without ``leaf_values`` — in this class itself, so the reference's constructor call
    ``Evaluator(model, device, cfg)`` (src/p2/rl/cfr_trainer.py:194-207) carries over unchanged."""

    def __init__(self, net, device, *, enforce_zero_sum: bool | None = None,
                 autocast_dtype: torch.dtype | None = None) -> None:
        self.net = net
        self.device = torch.device(device)
        # the reference reads the flag off the network (cfr_evaluator.py:970)
        self.enforce_zero_sum = bool(getattr(net, "enforce_zero_sum", False)) if enforce_zero_sum is None \
            else bool(enforce_zero_sum)
        self.autocast_dtype = autocast_dtype
        self._cached_for = None
        self._cached = None
        call = net.forward if isinstance(net, torch.nn.Module) else net
        self._policy_keyword = _accepts_keyword(call, "include_policy")

    def _run(self, feats, include_policy: bool):
        if hasattr(self.net, "eval"):
            self.net.eval()
        kw = {"include_policy": include_policy} if self._policy_keyword else {}
        if self.autocast_dtype is not None:
            with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                return self.net(feats, **kw)
        return self.net(feats, **kw)

    @torch.no_grad()
    def policy_logits(self, beliefs: torch.Tensor, rows: torch.Tensor, ev) -> torch.Tensor:
        """[K, 1326, actions] logits of the network at node rows ``rows`` (cfr_evaluator.py:305-319);
        zeros — a uniform policy over the legal actions — for a network without a policy head."""
        feats = ev.feature_encoder.encode(beliefs, indices=rows)
        logits = getattr(self._run(feats, True), "policy_logits", None) if self._policy_keyword else None
        if logits is None:
            return torch.zeros(rows.numel(), NUM_HANDS, ev.num_actions, dtype=torch.float32, device=self.device)
        return logits.reshape(rows.numel(), NUM_HANDS, ev.num_actions)

    @torch.no_grad()
    def leaf_values(self, beliefs: torch.Tensor, rows: torch.Tensor, ev) -> torch.Tensor:
        # Context and board of a leaf are public state: encoded once per subgame, only the ranges
        # change from iteration to iteration (the reference re-encodes every time).
        key = (id(ev), ev.subgame_serial, rows.data_ptr(), rows.numel())
        beliefs = beliefs.contiguous()
        if self._cached_for != key:
            self._cached = ev.feature_encoder.encode_rows(beliefs, rows, ev.new_street_mask[rows])
            self._cached_for = key
        c = self._cached
        feats = MLPFeatures(context=c.context, street=c.street, to_act=c.to_act, board=c.board,
                            beliefs=beliefs.reshape(beliefs.shape[0], -1))
        return self._run(feats, False).hand_values

    @torch.no_grad()
    def leaf_values_from_nodes(self, table: torch.Tensor, rows: torch.Tensor, ev) -> torch.Tensor:
        """The same answer from the whole node table ``table`` [total, 2, 1326]: for a network that
        offers ``forward_input`` / ``static_input_columns`` the input matrix is kept for the subgame,
        the leaves' ranges are written into it by one kernel in the network's dtype, and the answer is
        returned in that dtype (the evaluator converts while it stores).  Other networks get the
        gathered ranges through ``leaf_values``."""
        net = self.net
        if not (hasattr(net, "forward_input") and hasattr(net, "static_input_columns")):
            return self.leaf_values(table[rows], rows, ev)
        key = (id(ev), ev.subgame_serial, rows.data_ptr(), rows.numel(), "input")
        if self._cached_for != key:
            c = ev.feature_encoder.encode_rows(table[rows], rows, ev.new_street_mask[rows])
            feats = MLPFeatures(context=c.context, street=c.street, to_act=c.to_act, board=c.board,
                                beliefs=c.beliefs.reshape(rows.numel(), -1))
            self._cached = net.static_input_columns(feats, self.autocast_dtype or torch.float32)
            self._cached_for = key
        x = ev.gather_leaf_rows(table, rows, self._cached)
        if hasattr(net, "eval"):
            net.eval()
        if self.autocast_dtype is not None:
            with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                return net.forward_input(x).hand_values
        return net.forward_input(x).hand_values


class ChanceLeafModel:
    """Evaluator leaf protocol on top of a value network and the chance nodes (one card, flop)."""

    def __init__(self, net, device, *, enforce_zero_sum: bool = False, autocast_dtype: torch.dtype | None = None,
                 max_samples_per_call: int = 1 << 19) -> None:
        self.net = net
        self.device = torch.device(device)
        self.enforce_zero_sum = enforce_zero_sum
        self.autocast_dtype = autocast_dtype
        self.max_samples_per_call = int(max_samples_per_call)
        self.helper = ChanceNodeHelper(self.device, torch.float32, 2, net, autocast_dtype=autocast_dtype)
        self._plan_for = None
        self._plan = None

    def _make_plan(self, rows: torch.Tensor, ev):
        """Static split of the evaluator's model rows (the tree does not change between iterations)."""
        r = rows.cpu().numpy()
        tree = ev.tree
        board = tree.board[tree.root_index[r]]
        on_board = (board >= 0).sum(axis=1)
        flop = tree.new_street_mask[r] & (on_board == 0)      # preflop betting closed: three cards come
        chance = tree.new_street_mask[r] & (on_board < 5) & ~flop
        dev = self.device
        plan = SimpleNamespace(
            direct=torch.from_numpy(np.nonzero(~chance)[0]).to(dev),
            chance=torch.from_numpy(np.nonzero(chance)[0]).to(dev),
            flop=torch.from_numpy(np.nonzero(flop)[0]).to(dev),
            board=torch.from_numpy(board).to(dev),
            street=ev.env.street[rows].to(torch.long),
            to_act=ev.env.to_act[rows].to(torch.long),
            cards=int(on_board[chance][0]) if chance.any() and (on_board[chance] == on_board[chance][0]).all() else None,
        )
        return plan

    def _features(self, beliefs: torch.Tensor, plan, sel: torch.Tensor | None = None) -> MLPFeatures:
        k = beliefs.shape[0]
        f = MLPFeatures(context=torch.zeros(k, 1, dtype=torch.float32, device=self.device), street=plan.street,
                        to_act=plan.to_act, board=plan.board, beliefs=beliefs.reshape(k, -1))
        return f if sel is None else f[sel]

    @torch.no_grad()
    def leaf_values(self, beliefs: torch.Tensor, rows: torch.Tensor, ev) -> torch.Tensor:
        key = (id(ev), ev.subgame_serial, rows.data_ptr(), rows.numel())
        if self._plan_for != key:
            self._plan, self._plan_for = self._make_plan(rows, ev), key
        plan = self._plan
        beliefs = beliefs.contiguous().float()
        out = torch.empty_like(beliefs)
        if plan.direct.numel():
            feats = self._features(beliefs, plan, plan.direct)
            if hasattr(self.net, "eval"):
                self.net.eval()
            if self.autocast_dtype is not None:
                with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                    hv = self.net(feats).hand_values
            else:
                hv = self.net(feats).hand_values
            out.index_copy_(0, plan.direct, hv.to(out.dtype))
        if plan.chance.numel():
            feats = self._features(beliefs, plan)
            per_state = 52 - (plan.cards if plan.cards is not None else 0)
            step = max(1, self.max_samples_per_call // per_state)
            for lo in range(0, plan.chance.numel(), step):
                sel = plan.chance[lo:lo + step]
                ev_chance = self.helper.single_card_chance_values(sel, feats, beliefs, plan.board,
                                                                  cards_on_board=plan.cards, check_rows=False)
                out.index_copy_(0, sel, ev_chance.to(out.dtype))
        if plan.flop.numel():
            feats = self._features(beliefs, plan)
            flops_per_call = self.helper.FLOP_SAMPLE_SIZE or self.helper.FLOP_CHUNK_SIZE
            step = max(1, self.max_samples_per_call // flops_per_call)
            for lo in range(0, plan.flop.numel(), step):
                sel = plan.flop[lo:lo + step]
                out.index_copy_(0, sel, self.helper.flop_chance_values(sel, feats, beliefs).to(out.dtype))
        return out
