"""CPU: the C-ABI library loads and exports every symbol include/p2hip.h declares; the
product package never touches the oracle."""
import os
import re

from tests.conftest import ROOT


def header_symbols():
    text = open(os.path.join(ROOT, "include", "p2hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(p2hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from poker2_amd import _lib
    lib = _lib.load()
    syms = header_symbols()
    assert len(syms) >= 30
    for name in syms:
        assert hasattr(lib, name), name
    assert sorted(_lib.declared_symbols()) == syms
    assert lib.p2hip_abi_version() >= 1
    assert lib.p2hip_showdown_table_bytes() % 256 == 0


def test_argument_errors_without_a_gpu():
    from poker2_amd import _lib
    lib = _lib.load()
    # negative sizes / null pointers are rejected before any launch
    assert lib.p2hip_unblocked_mass(None, -1, None, None) == 1
    assert lib.p2hip_unblocked_mass(None, 3, None, None) == 1
    assert lib.p2hip_rank7_cards(None, 3, 5, None, None) == 1
    assert lib.p2hip_dcfr_update(None, None, None, None, None, None, None, 3, 1, 0, None, None) == 1
    assert lib.p2hip_unblocked_mass(None, 0, None, None) == 0


def test_product_never_imports_oracle():
    pkg = os.path.join(ROOT, "poker2_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.replace("oracle/", "oracle/"), f


def test_wrappers_fail_loudly_without_gpu():
    import pytest
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from poker2_amd import fused_cfr_hip, rules_hip
    assert not fused_cfr_hip.triton_is_available()
    with pytest.raises((RuntimeError, ValueError)):
        rules_hip.rank_7_cards_single_batch_triton(torch.zeros(4, 7, dtype=torch.int16))
    with pytest.raises((RuntimeError, ValueError)):
        fused_cfr_hip.unblocked_mass_triton(torch.zeros(2, 1326))
    # the chance-node and data-generation wrappers have no CPU path either
    from types import SimpleNamespace
    from poker2_amd import chance_node_helper as CH
    from poker2_amd.rebel_feature_encoder import RebelFeatureEncoder
    z = torch.zeros(1, 2, 1326)
    with pytest.raises((RuntimeError, ValueError)):
        CH.chance_expand(z, torch.zeros(1, dtype=torch.long), torch.full((1, 5), -1))
    with pytest.raises((RuntimeError, ValueError)):
        CH.chance_mean(z, torch.tensor([0, 1]))
    with pytest.raises((RuntimeError, ValueError)):
        CH.flop_expand(z, torch.zeros(1, dtype=torch.long), torch.tensor([[0, 1, 2]]))
    with pytest.raises((RuntimeError, ValueError)):
        CH.perm_mean(torch.zeros(1, 1, 2, 1326), torch.arange(1326)[None], torch.ones(1))
    env = SimpleNamespace(**{k: torch.zeros(1, dtype=torch.long) for k in ("to_act", "button", "pot", "actions_this_round")},
                          starting_stacks=torch.ones(1, 2, dtype=torch.long), committed=torch.zeros(1, 2, dtype=torch.long),
                          board_indices=torch.full((1, 5), -1), last_board_indices=torch.full((1, 5), -1))
    with pytest.raises((RuntimeError, ValueError)):
        RebelFeatureEncoder(env).encode(z)
    helper = CH.ChanceNodeHelper(torch.device("cpu"), torch.float32, 2, model=None, autocast_dtype=None)
    with pytest.raises((RuntimeError, ValueError)):
        helper.flop_chance_values(torch.zeros(1, dtype=torch.long), None, z)


def test_argument_guards_hold_under_python_O():
    """The wrappers' argument checks are what keeps a wrong shape from becoming a GPU memory fault;
    they must not be compiled out by ``python -O`` the way ``assert`` is."""
    import subprocess
    import sys
    code = ("import numpy as np\n"
            "from poker2_amd._guards import require\n"
            "from poker2_amd.tree import RootStates, build_sparse_tree\n"
            "assert False, 'asserts are off under -O, so this line must not raise'\n"
            "try:\n"
            "    require(1 + 1 == 3, 'refused')\n"
            "except AssertionError as e:\n"
            "    assert str(e) == 'refused'\n"
            "else:\n"
            "    raise SystemExit(3)\n"
            "try:\n"
            "    build_sparse_tree(RootStates.at_round_start(3, np.zeros(0), np.zeros((0, 2)), np.zeros((0, 5))), [0.5], 2)\n"
            "except AssertionError:\n"
            "    raise SystemExit(0)\n"
            "raise SystemExit(4)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-O", "-c", code], cwd=root, capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr[-2000:]
    # no plain assert is left in the package's modules
    import glob
    import re
    left = [p for p in glob.glob(os.path.join(root, "poker2_amd", "*.py"))
            if re.search(r"^\s*assert\b", open(p).read(), re.M)]
    assert left == [], left


def test_bench_refuses_more_than_one_gpu_and_has_the_contract_flags():
    """bench.py measures one GPU; asked for more it says so and exits without touching a GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "bench.py", "--gpus", "2", "--steps", "1", "--warmup", "0"], cwd=root,
                         capture_output=True, text=True, timeout=300)
    assert res.returncode == 2 and "ONE GPU" in res.stderr and res.stdout.strip() == ""
    helptext = subprocess.run([sys.executable, "bench.py", "--help"], cwd=root, capture_output=True, text=True,
                              timeout=300).stdout
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in helptext
