"""GPU: the product's per-operation entry points (poker2_amd.fused_cfr_hip -> libp2hip.so) against
outputs of the reference's own Triton kernels (tests/golden/fused_ops_golden.npz, written under
Triton's CPU interpreter).  Same seeded inputs, same call sequence as the fixture's writer.
Tolerance 1e-5 relative + 1e-6 absolute per element."""
import os

import numpy as np
import pytest

from tests import fused_op_cases as C
from tests.test_oracle_fused_ops import check_against_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def golden(golden_dir):
    return np.load(os.path.join(golden_dir, "fused_ops_golden.npz"))


@pytest.mark.parametrize("name", C.NAMES)
def test_product_matches_reference_kernel_outputs(golden, name):
    import torch

    from poker2_amd import fused_cfr_hip as F
    got = C.torch_ops(name, C.inputs(name), F, torch.device("cuda:0"))
    torch.cuda.synchronize()
    check_against_golden(golden, name, {k: v.detach().cpu().numpy() for k, v in got.items()})
