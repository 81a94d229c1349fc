"""GPU parity: every per-operation HIP kernel against the CPU oracle, called through the
reference-named Python wrappers (which call the C ABI of libp2hip.so).

Shapes and seeds follow the reference's tests/test_fused_cfr_triton.py; tolerances are the
ones that file uses (rtol 1e-5 / atol 1e-6 for element-wise work)."""
import numpy as np
import pytest
import torch

from oracle import cfr_ops as O
from oracle import unblocked as OU
from tests.helpers import H, random_tree

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6


@pytest.fixture(scope="module")
def F():
    from poker2_amd import fused_cfr_hip
    assert fused_cfr_hip.triton_is_available(), "libp2hip.so / GPU missing"
    return fused_cfr_hip


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def close(a: torch.Tensor, b: np.ndarray, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(a.cpu().numpy(), b, rtol=rtol, atol=atol)


@pytest.mark.parametrize("cfr_type", ["discounted", "discounted_plus", "standard"])
@pytest.mark.parametrize("cfr_plus", [False, True])
@pytest.mark.parametrize("t", [0, 1, 7, 50])
def test_dcfr_update(F, cfr_type, cfr_plus, t):
    rng = np.random.default_rng(0xC0FFEE + t + int(cfr_plus))
    shape = (37, H)
    cumul = rng.standard_normal(shape).astype(np.float32)
    weight = (rng.random(shape) * 5).astype(np.float32)
    regrets = (rng.standard_normal(shape) * 0.1).astype(np.float32)
    apply = cfr_type != "standard"
    ec, ew, ep = O.dcfr_update(cumul, weight, regrets, t, 1.5, 0.5, apply, cfr_plus)
    c, w, r = dev(cumul), dev(weight), dev(regrets)
    pos = torch.empty_like(c)
    F.fused_dcfr_update_(c, w, r, t, F.CFRType[cfr_type], 1.5, 0.5, cfr_plus, positive_regrets_out=pos)
    close(c, ec); close(w, ew); close(pos, ep)
    # bit-exact: same operation order and correctly rounded division
    assert np.array_equal(c.cpu().numpy(), ec) and np.array_equal(w.cpu().numpy(), ew)


def test_dcfr_update_linear_rejected(F):
    x = torch.zeros(2, H, device="cuda")
    with pytest.raises(NotImplementedError):
        F.fused_dcfr_update_(x, x.clone(), x.clone(), 3, F.CFRType.linear, 1.5, 0.0, False)
    with pytest.raises(ValueError):
        c = torch.zeros(2, H)
        F.fused_dcfr_update_(c, c.clone(), c.clone(), 3, F.CFRType.discounted, 1.5, 0.0, False)


@pytest.mark.parametrize("three_d", [True, False])
def test_block_and_normalize(F, three_d):
    rng = np.random.default_rng(7)
    n = 29
    target = rng.random((n, 2, H) if three_d else (n, H)).astype(np.float32)
    allowed = rng.random((n, H)) > 0.3
    allowed[3] = False  # a fully blocked row falls back
    prob = rng.random((n, H)).astype(np.float32)
    if three_d:
        target[5, 1] = 0.0  # zero row falls back
    exp = O.block_and_normalize(target, allowed, prob)
    t = dev(target)
    F.fused_block_and_normalize_beliefs_(t, dev(allowed), dev(prob))
    close(t, exp)


def test_regret_matching_divide(F):
    rng = np.random.default_rng(11)
    pos = rng.random((31, H)).astype(np.float32)
    den = rng.random((31, H)).astype(np.float32)
    den[::3] = 0.0
    uni = rng.random((31, H)).astype(np.float32)
    out = torch.empty(31, H, device="cuda")
    F.fused_regret_matching_divide_(dev(pos), dev(den), dev(uni), out)
    close(out, O.regret_matching_divide(pos, den, uni))


def test_weight_child_values(F):
    rng = np.random.default_rng(13)
    m = 23
    v = rng.standard_normal((m, 2, H)).astype(np.float32)
    pa = rng.integers(0, 2, m).astype(np.int64)
    ph = rng.random((m, H)).astype(np.float32)
    po = rng.random((m, H)).astype(np.float32)
    out = torch.empty(m, 2, H, device="cuda")
    F.fused_weight_child_values(dev(v), dev(pa), dev(ph), dev(po), out)
    close(out, O.weight_child_values(v, pa, ph, po))


def test_update_average_values(F):
    rng = np.random.default_rng(17)
    avg = rng.standard_normal((40, 2, H)).astype(np.float32)
    lat = rng.standard_normal((40, 2, H)).astype(np.float32)
    a = dev(avg)
    F.fused_update_average_values_(a, dev(lat), 9.0, 16.0)
    close(a, O.update_average_values(avg, lat, 9.0, 16.0))


@pytest.mark.parametrize("enforce", [False, True])
@pytest.mark.parametrize("with_ignore", [False, True])
def test_avg_values_zero_sum(F, enforce, with_ignore):
    rng = np.random.default_rng(19)
    n = 21
    avg = rng.standard_normal((n, 2, H)).astype(np.float32)
    lat = rng.standard_normal((n, 2, H)).astype(np.float32)
    bel = rng.random((n, 2, H)).astype(np.float32)
    bel /= bel.sum(-1, keepdims=True)
    ign = rng.random(n) > 0.5 if with_ignore else None
    exp = O.avg_values_zero_sum(avg, lat, bel, 4.0, 9.0, enforce, ign)
    a = dev(avg)
    sc = lambda v: torch.tensor(v, dtype=torch.float32, device="cuda")  # noqa: E731
    F.fused_avg_values_zero_sum_(a, dev(lat), dev(bel), sc(4.0), sc(9.0), sc(1.0 / 13.0), enforce,
                                 ignore_mask=dev(ign) if with_ignore else None)
    close(a, exp, rtol=1e-5, atol=2e-6)
    if enforce and not with_ignore:
        v = a.cpu().numpy()
        zs = (v * bel).sum(-1).sum(-1)
        assert np.abs(zs).max() < 1e-4


def _tree(seed, n_roots=6, depth=3):
    return random_tree(np.random.default_rng(seed), n_roots, depth)


def test_regret_tail(F):
    rng = np.random.default_rng(19)
    tr = _tree(1)
    total, top, bottom = tr["total"], tr["top"], tr["bottom"]
    ach = rng.standard_normal((total, 2, H)).astype(np.float32)
    av = rng.standard_normal((top, H)).astype(np.float32)
    sw = rng.standard_normal((top, H)).astype(np.float32)
    reg = torch.zeros(total, H, device="cuda")
    F.fused_regret_tail_(reg, dev(ach), dev(av), dev(sw), dev(tr["parent_index"]), dev(tr["prev_actor"]), bottom)
    close(reg, O.regret_tail(ach, av, sw, tr["parent_index"], tr["prev_actor"], bottom))


def test_average_policy_mix(F):
    rng = np.random.default_rng(23)
    tr = _tree(2)
    total, bottom = tr["total"], tr["bottom"]
    reach = rng.random((total, 2, H)).astype(np.float32)
    reach_avg = rng.random((total, 2, H)).astype(np.float32)
    reach[:, :, ::5] = 0.0
    reach_avg[:, :, ::5] = 0.0  # exercise the un-weighted fallback
    pol = rng.random((total, H)).astype(np.float32)
    pavg = rng.random((total, H)).astype(np.float32)
    exp = O.average_policy_mix(pavg, pol, reach, reach_avg, tr["to_act"], tr["parent_index"], 3.0, 2.0, bottom)
    a = dev(pavg)
    F.fused_average_policy_mix_(a, dev(pol), dev(reach), dev(reach_avg), dev(tr["to_act"]), dev(tr["parent_index"]),
                                3.0, 2.0, bottom)
    close(a, exp)


def test_parent_sum_divide_and_sibling_sum(F):
    rng = np.random.default_rng(43)
    tr = _tree(3, n_roots=9, depth=3)
    total, top, bottom = tr["total"], tr["top"], tr["bottom"]
    nchild = total - bottom
    values = rng.standard_normal((total, H)).astype(np.float32)
    co, cc = tr["child_offsets"][:top].copy(), tr["child_count"][:top].copy()
    ps = F.fused_parent_sum(dev(values), dev(co), dev(cc))
    exp_ps = O.parent_sum(values, co, cc)
    close(ps, exp_ps, atol=1e-5)
    ss = F.fused_sibling_sum(dev(values), dev(co), dev(cc), bottom, nchild)
    close(ss, O.sibling_sum(values, co, cc, bottom, nchild), atol=1e-5)
    pos = rng.random((nchild, H)).astype(np.float32)
    fb = rng.random((nchild, H)).astype(np.float32)
    psum = np.abs(exp_ps)
    psum[:, ::4] = 0.0
    out = torch.empty(nchild, H, device="cuda")
    pidx = tr["parent_index"][bottom:].copy()
    F.fused_divide_by_parent_sum_(dev(pos), dev(fb), dev(psum), dev(pidx), out)
    close(out, O.divide_by_parent_sum(pos, fb, psum, pidx), rtol=1e-5, atol=1e-6)
    # in place (out aliases pos and fallback), as update_average_policy uses it
    buf = dev(pos)
    F.fused_divide_by_parent_sum_(buf, buf, dev(psum), dev(pidx), buf, eps=1e-5)
    close(buf, O.divide_by_parent_sum(pos, pos, psum, pidx, eps=1e-5))


def test_model_values_mix(F):
    rng = np.random.default_rng(41)
    h = rng.standard_normal((80, 2, H)).astype(np.float32)
    l = rng.standard_normal((80, 2, H)).astype(np.float32)
    out = F.fused_model_values_mix(dev(h), dev(l), 5.0, 3.0)
    close(out, O.model_values_mix(h, l, 5.0, 3.0))
    bel = rng.random((80, 2, H)).astype(np.float32)
    bel /= bel.sum(-1, keepdims=True)
    sc = lambda v: torch.tensor(v, dtype=torch.float32, device="cuda")  # noqa: E731
    for enforce in (False, True):
        o = torch.empty(80, 2, H, device="cuda")
        F.fused_model_values_mix_zero_sum(dev(h), dev(l), dev(bel), sc(8.0 / 3.0), sc(5.0 / 3.0), o, enforce)
        close(o, O.model_values_mix_zero_sum(h, l, bel, 5.0, 3.0, enforce), rtol=1e-5, atol=2e-6)


def test_weighted_parent_sum(F):
    rng = np.random.default_rng(71)
    tr = _tree(4, n_roots=5, depth=3)
    total = tr["total"]
    offs = tr["depth_offsets"]
    values = rng.standard_normal((total, 2, H)).astype(np.float32)
    ph = rng.random((total, H)).astype(np.float32)
    po = rng.random((total, H)).astype(np.float32)
    exp = values.copy()
    v = dev(values)
    for d in range(len(offs) - 3, -1, -1):
        base, end = offs[d], offs[d + 1]
        co, cc = tr["child_offsets"][base:end].copy(), tr["child_count"][base:end].copy()
        exp = O.weighted_parent_sum(exp, tr["prev_actor"], ph, po, co, cc, base)
        F.fused_weighted_parent_sum(v, dev(tr["prev_actor"]), dev(ph), dev(po), dev(co), dev(cc), base)
    close(v, exp, rtol=1e-4, atol=1e-5)


def test_reach_weights_and_deep_beliefs(F):
    rng = np.random.default_rng(73)
    tr = _tree(5, n_roots=4, depth=3)
    total, n = tr["total"], tr["bottom"]
    offs = tr["depth_offsets"]
    reach = rng.random((total, 2, H)).astype(np.float32)
    pol = rng.random((total, H)).astype(np.float32)
    allowed = rng.random((total, H)) > 0.2
    exp = reach.copy()
    r = dev(reach)
    for d in range(len(offs) - 2):
        s, e = offs[d + 1], offs[d + 2]
        exp = O.reach_weights_depth(exp, pol, allowed, tr["parent_index"], tr["prev_actor"], s, e)
        F.fused_reach_weights_depth_(r, dev(pol), dev(allowed), dev(tr["parent_index"]), dev(tr["prev_actor"]), s, e)
    close(r, exp)
    bel = rng.random((total, 2, H)).astype(np.float32)
    prob = rng.random((total, H)).astype(np.float32)
    exp[n + 1] = 0.0  # a dead node falls back to allowed_prob
    expb = O.deep_beliefs(bel, bel, exp, prob, tr["root_index"], n)
    b = dev(bel)
    F.fused_deep_beliefs_(b, b, dev(exp), dev(prob), dev(tr["root_index"]), num_roots=n)
    close(b, expb, rtol=1e-5, atol=1e-6)


def test_sample_snapshot(F):
    rng = np.random.default_rng(5)
    pol = rng.random((12, H)).astype(np.float32)
    smp = rng.random((12, H)).astype(np.float32)
    ts = np.array([3, 4, 3, 9, 3, 3, 1, 0, 3, 2, 3, 7], dtype=np.int64)
    s = dev(smp)
    F.fused_sample_snapshot_(s, dev(pol), dev(ts), torch.tensor(3, device="cuda"))
    exp = np.where((ts == 3)[:, None], pol, smp)
    assert np.array_equal(s.cpu().numpy(), exp)


# ---- unblocked mass ---------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(1, H), (17, H), (5, 2, H)])
def test_unblocked_mass(F, shape):
    rng = np.random.default_rng(29)
    t = rng.random(shape).astype(np.float32)
    out = F.unblocked_mass_triton(dev(t))
    exp = OU.calculate_unblocked_mass(t)
    close(out, exp, rtol=1e-6, atol=1e-5)
    from poker2_amd.card_utils import calculate_unblocked_mass
    close(calculate_unblocked_mass(dev(t)), exp, rtol=1e-6, atol=1e-5)


def test_unblocked_mass_known_answers(F):
    u = np.full((1, H), 1.0 / H, dtype=np.float32)
    out = F.unblocked_mass_triton(dev(u)).cpu().numpy()
    np.testing.assert_allclose(out, 0.9238311052322388, rtol=1e-6)  # 1225/1326
    d = np.zeros((1, H), dtype=np.float32)
    d[0, 0] = 1.0  # combo (0,1)
    out = F.unblocked_mass_triton(dev(d)).cpu().numpy()[0]
    from oracle.cards import hand_combos
    cm = hand_combos()
    shares = (cm[:, 0] <= 1) | (cm[:, 1] <= 1)
    assert np.array_equal(out, np.where(shares, 0.0, 1.0).astype(np.float32))
    z = np.zeros((3, H), dtype=np.float32)
    assert np.array_equal(F.unblocked_mass_triton(dev(z)).cpu().numpy(), z)


def test_unblocked_mass_opp_at_parents_and_ratio(F):
    rng = np.random.default_rng(47)
    total, top = 33, 12
    bel = rng.random((total, 2, H)).astype(np.float32)
    to_act = rng.integers(0, 2, total).astype(np.int64)
    out = F.unblocked_mass_opp_at_parents_triton(dev(bel), dev(to_act), top)
    exp = OU.calculate_unblocked_mass(bel[np.arange(top), 1 - to_act[:top]])
    close(out, exp, rtol=1e-6, atol=1e-5)

    nchild = 40
    actor = rng.random((top, H)).astype(np.float32)
    actor /= actor.sum(-1, keepdims=True)
    actor[2] = 0.0  # zero denominator row -> ratio 0
    pidx = rng.integers(0, top, nchild).astype(np.int64)
    pol = rng.random((nchild, H)).astype(np.float32)
    numer = (actor[pidx] * pol).astype(np.float32)
    out = F.unblocked_mass_ratio_indirect_triton(dev(numer), dev(actor), dev(pidx))
    exp = OU.unblocked_mass_ratio(numer, actor, 1e-5, pidx)
    close(out, exp, rtol=1e-4, atol=1e-6)
    out2 = F.unblocked_mass_ratio_triton(dev(numer), dev(actor[pidx]))
    close(out2, exp, rtol=1e-4, atol=1e-6)


def test_unblocked_mass_grid_stride_ragged_and_empty(F):
    """More rows than one pass of the persistent kernels covers (4 rows x 1024 workgroups),
    a row count that is not a multiple of the group size, an odd ratio count, and no rows."""
    rng = np.random.default_rng(53)
    rows = 2 * 4096 + 3
    t = rng.random((rows, H)).astype(np.float32)
    t[5] = 0.0
    out = F.unblocked_mass_triton(dev(t))
    close(out, OU.calculate_unblocked_mass(t), rtol=1e-6, atol=1e-4)
    n = 2 * 2048 + 1
    numer = (t[:n] * rng.random((n, 1)).astype(np.float32)).astype(np.float32)
    pidx = rng.integers(0, rows, n).astype(np.int64)
    out = F.unblocked_mass_ratio_indirect_triton(dev(numer), dev(t), dev(pidx))
    close(out, OU.unblocked_mass_ratio(numer, t, 1e-5, pidx), rtol=1e-4, atol=1e-6)
    empty = torch.zeros(0, H, device="cuda")
    assert F.unblocked_mass_triton(empty).shape == (0, H)
    assert F.unblocked_mass_ratio_triton(empty, empty).shape == (0, H)


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 7, 1030])
def test_unblocked_mass_at_every_buffer_alignment_and_ragged_row_counts(rows):
    """Through the C ABI with buffers at several offsets inside a 128-byte line (8-byte alignment is all the
    entry points ask for): the oracle's values, nothing written outside the output rows, bit-identical
    results whatever the alignment, for row counts that leave the last group of four rows ragged, and
    for rows picked by player."""
    from poker2_amd import _lib
    rng = np.random.default_rng(600 + rows)
    t = rng.random((rows, H)).astype(np.float32)
    t[rows // 2, ::3] = 0.0
    exp = OU.calculate_unblocked_mass(t)
    stream = _lib.stream_ptr()
    results = []
    for offset in (0, 2, 4, 8, 12, 28):               # in floats
        src = torch.zeros(rows * H + 64, device="cuda")
        dst = torch.full((rows * H + 64,), -7.0, device="cuda")
        a, b = src[offset:offset + rows * H], dst[offset:offset + rows * H]
        a.copy_(torch.from_numpy(t).reshape(-1))
        _lib.call("p2hip_unblocked_mass", a.data_ptr(), rows, b.data_ptr(), stream)
        torch.cuda.synchronize()
        assert (dst[:offset] == -7.0).all() and (dst[offset + rows * H:] == -7.0).all()   # nothing outside
        results.append(b.reshape(rows, H).cpu().numpy())
        close(b.reshape(rows, H), exp, rtol=1e-6, atol=1e-5)
    for r in results[1:]:
        assert np.array_equal(r, results[0])
    # by player: rows 2 r + (to_act[r] ^ flip) of a [rows, 2, H] tensor
    bel = rng.random((rows, 2, H)).astype(np.float32)
    to_act = rng.integers(0, 2, rows).astype(np.int64)
    exp2 = OU.calculate_unblocked_mass(bel[np.arange(rows), 1 - to_act])
    got = []
    for offset in (0, 2):
        dst = torch.full((rows * H + 64,), -7.0, device="cuda")
        b = dst[offset:offset + rows * H]
        _lib.call("p2hip_unblocked_mass_by_player", dev(bel).data_ptr(), dev(to_act).data_ptr(), rows, 1,
                  b.data_ptr(), stream)
        torch.cuda.synchronize()
        assert (dst[:offset] == -7.0).all() and (dst[offset + rows * H:] == -7.0).all()
        got.append(b.reshape(rows, H).cpu().numpy())
        close(b.reshape(rows, H), exp2, rtol=1e-6, atol=1e-5)
    assert np.array_equal(got[0], got[1])


def test_tscalars_update_fills_every_scalar_with_one_array_behind_them(F):
    """TScalars.update (fused_cfr_triton.py:2131-2158): every 0-D tensor holds what the reference's fills
    would leave, the de-averaging pair keeps its last values while mix_new is zero, and on the GPU all of
    them are views of one array (refreshed by a launch or two instead of eleven)."""
    sc = F.TScalars(torch.device("cuda"))
    expect = {}

    def check(t, alpha, beta, old, new):
        sc.update(t, alpha, beta, old, new)
        (an, ad), (bn, bd) = F.discount_pair(t, alpha), F.discount_pair(t, beta)
        total = float(old) + float(new)
        expect.update(t_alpha_num=an, t_alpha_den=ad, t_beta_num=bn, t_beta_den=bd, mix_old=old, mix_new=new,
                      mix_total=total, mix_inv_total=1.0 / total if total else 1.0)
        if new != 0.0:
            expect.update(mix_onon=total / new, mix_oon=old / new)
        for name, value in expect.items():
            got = getattr(sc, name)
            assert got.dim() == 0 and got.dtype == torch.float32
            assert float(got) == np.float32(value), (name, t)
        assert sc.t_tensor.dim() == 0 and sc.t_tensor.dtype == torch.int64 and int(sc.t_tensor) == t

    expect.update(mix_onon=0.0, mix_oon=0.0)
    check(0, 1.5, -1.0, 1.0, 0.0)          # mix_new = 0: the pair stays as it was
    check(7, 1.5, 0.0, 10.5, 3.0)
    check(8, 1.5, 0.5, 4.0, 0.0)           # and keeps the values of t = 7 here
    check(50, 2.0, -1.0, 0.0, 2.0)
    base = sc.floats.data_ptr()
    assert [getattr(sc, n).data_ptr() - base for n in F.TScalars._NAMES] == [4 * k for k in range(10)]
    assert sc.t_tensor.data_ptr() == sc.ints.data_ptr()


def test_stream_probe_moves_what_it_says():
    """The measurement aid behind bench.py's flat-stream figure: every output array holds the sum of the input
    arrays plus its own number (so every load and every store happens), and unsupported mixes are refused."""
    from poker2_amd import _lib
    pairs = 1000 * 256 + 77
    rng = np.random.default_rng(3)
    src = torch.from_numpy(rng.random((5, pairs, 2)).astype(np.float32)).cuda()
    dst = torch.full((7, pairs, 2), -1.0, device="cuda")
    acc = torch.tensor([1.0, 2.0], device="cuda").expand(pairs, 2).clone()
    for k in range(5):
        acc = acc + src[k]
    for non_temporal in (0, 1):
        dst.fill_(-1.0)
        _lib.call("p2hip_stream_probe", src.data_ptr(), dst.data_ptr(), pairs, 5, 7, non_temporal, _lib.stream_ptr())
        torch.cuda.synchronize()
        for k in range(7):
            exp = acc.clone()
            exp[:, 0] += float(k)
            assert torch.equal(dst[k], exp)
    code = _lib.load().p2hip_stream_probe(src.data_ptr(), dst.data_ptr(), pairs, 3, 3, 0, _lib.stream_ptr())
    assert code != 0


def test_wrappers_refuse_arguments_that_would_index_out_of_bounds(F):
    """Sizes, dtypes and row bounds the kernels index with are checked on the host (and stay
    checked under ``python -O``): none of these calls may reach the GPU."""
    rng = np.random.default_rng(77)
    tr = random_tree(rng, 3, 2)
    total, top, bottom = tr["total"], tr["top"], tr["bottom"]
    reach = torch.ones(total, 2, H, device="cuda")
    policy = torch.rand(total, H, device="cuda")
    allowed = torch.ones(total, H, dtype=torch.bool, device="cuda")
    pidx, pa, to_act = dev(tr["parent_index"]), dev(tr["prev_actor"]), dev(tr["to_act"])
    co, cc = dev(tr["child_offsets"][:top].copy()), dev(tr["child_count"][:top].copy())
    one = torch.ones((), device="cuda")
    bad = [
        lambda: F.fused_reach_weights_depth_(reach, policy, allowed, pidx.int(), pa, bottom, total),     # int32 indices
        lambda: F.fused_reach_weights_depth_(reach, policy, allowed, pidx, pa, bottom, total + 5),       # rows past the end
        lambda: F.fused_reach_weights_depth_(reach.double(), policy, allowed, pidx, pa, bottom, total),  # not fp32
        lambda: F.fused_regret_tail_(torch.zeros(total, H, device="cuda"), reach, policy[:top].contiguous(),
                                     policy[:top].contiguous(), pidx, pa, total + 1),
        lambda: F.unblocked_mass_opp_at_parents_triton(reach, to_act, total + 1),
        lambda: F.fused_dcfr_update_with_tensors_(policy, policy[:-1].contiguous(), policy.clone(), one, one, one, one,
                                                  True, False),
        lambda: F.fused_update_average_values_with_tensors_(reach, reach[:-1].contiguous(), one, one, one),
        lambda: F.fused_update_average_values_with_tensors_(reach.half(), reach.half(), one, one, one),
        lambda: F.fused_sibling_sum(policy, co, cc, bottom, total - bottom + 10),
        lambda: F.fused_weighted_parent_sum(reach, pa, policy, policy, co, cc, total),
        lambda: F.fused_average_policy_mix_with_tensors_(policy, policy.clone(), reach, reach[:-1].contiguous(), to_act,
                                                         pidx, one, one, one, bottom),
        lambda: F.fused_deep_beliefs_(reach, reach, reach.clone(), policy, dev(tr["root_index"]).int(), bottom),
        lambda: F.fused_sample_snapshot_(policy, policy.clone(), to_act[:-1].contiguous(), torch.zeros((), dtype=torch.long,
                                                                                                      device="cuda")),
    ]
    for i, call in enumerate(bad):
        with pytest.raises(AssertionError):
            call()
            pytest.fail(f"call {i} was not refused")
    torch.cuda.synchronize()
