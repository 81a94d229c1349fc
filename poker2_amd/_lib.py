"""ctypes binding of ``libp2hip.so`` (the only compute path of this package).

There is no fallback: if the library is missing or a call fails, an exception
is raised.  Tensors are passed as raw device pointers; launches go to torch's
current stream.
"""
from __future__ import annotations

import ctypes
import os

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libp2hip.so")

_lib: ctypes.CDLL | None = None

_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float

# name -> argument types (return type is int unless listed in _RESTYPE)
_SIGNATURES: dict[str, list] = {
    "p2hip_abi_version": [],
    "p2hip_device_count": [],
    "p2hip_error_string": [_I],
    "p2hip_rank7_cards": [_P, _I, _L, _P, _P],
    "p2hip_compare7_cards": [_P, _I, _L, _P, _P],
    "p2hip_rank7_planes": [_P, _L, _P, _I, _P],
    "p2hip_compare7_planes": [_P, _L, _P, _I, _P],
    "p2hip_showdown_table_bytes": [],
    "p2hip_showdown_setup": [_P, _I, _L, _I, _P, _P, _P, _P],
    "p2hip_showdown_setup_sorted": [_P, _P, _P, _P, _L, _P, _P, _P],
    "p2hip_showdown_both": [_P, _P, _P, _P, _P, _L, _P, _P],
    "p2hip_best_response_level": [_P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _P],
    "p2hip_upload_floats": [_P, _P, _I, _P],
    "p2hip_tree_node_columns": [],
    "p2hip_tree_legal": [_P, _L, _P, _I, _I, _I, _I, _P, _P, _P],
    "p2hip_tree_step": [_P, _L, _L, _P, _I, _I, _L, _I, _P, _P, _P],
    "p2hip_chance_expand": [_P, _P, _P, _L, _P, _L, _L, _P, _P, _P, _P],
    "p2hip_chance_expand_input": [_P, _P, _P, _L, _P, _L, _L, _P, _I, _P, _P, _P],
    "p2hip_flop_expand": [_P, _P, _L, _P, _L, _P, _P],
    "p2hip_perm_mean": [_P, _L, _L, _P, _I, _P, _I, _P, _P, _I, _P],
    "p2hip_chance_mean": [_P, _P, _L, _P, _P],
    "p2hip_orbit_mean": [_P, _L, _L, _P, _I, _P, _P, _I, _P],
    "p2hip_orbit_mean_static": [_P, _L, _L, _P, _I, _P, _I, _P],
    "p2hip_encode_context": [_P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _L, _P, _P, _P],
    "p2hip_bet_amounts": [_P, _P, _P, _P, _L, _P, _I, _P, _P],
    "p2hip_policy_targets": [_P, _P, _L, _P, _P, _P, _I, _P, _P],
    "p2hip_gather_leaf_rows": [_P, _P, _L, _L, _P, _I, _L, _P],
    "p2hip_scatter_leaf_rows": [_P, _I, _L, _P, _L, _P, _L, _P],
    "p2hip_unblocked_mass": [_P, _L, _P, _P],
    "p2hip_unblocked_mass_by_player": [_P, _P, _L, _I, _P, _P],
    "p2hip_unblocked_mass_ratio": [_P, _P, _P, _L, _F, _P, _P],
    "p2hip_unblocked_mass_ratio_of": [_P, _P, _P, _L, _F, _P, _P],
    "p2hip_dcfr_update": [_P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _P, _P],
    "p2hip_block_and_normalize": [_P, _P, _P, _L, _I, _F, _P],
    "p2hip_regret_matching_divide": [_P, _P, _P, _P, _L, _F, _P],
    "p2hip_weight_child_values": [_P, _P, _P, _P, _P, _L, _P],
    "p2hip_update_average_values": [_P, _P, _P, _P, _P, _L, _P],
    "p2hip_avg_values_zero_sum": [_P, _P, _P, _P, _P, _P, _P, _L, _I, _P],
    "p2hip_regret_tail": [_P, _P, _P, _P, _P, _P, _L, _L, _P],
    "p2hip_average_policy_mix": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _F, _P],
    "p2hip_parent_sum": [_P, _P, _P, _L, _P, _P],
    "p2hip_sibling_sum": [_P, _P, _P, _L, _L, _P, _P],
    "p2hip_divide_by_parent_sum": [_P, _P, _P, _P, _P, _L, _F, _P],
    "p2hip_model_values_mix": [_P, _P, _P, _P, _P, _L, _P],
    "p2hip_model_values_mix_zero_sum": [_P, _P, _P, _P, _P, _P, _L, _I, _P],
    "p2hip_weighted_parent_sum": [_P, _P, _P, _P, _P, _P, _L, _L, _P],
    "p2hip_reach_weights_depth": [_P, _P, _P, _P, _P, _L, _L, _P],
    "p2hip_deep_beliefs": [_P, _P, _P, _P, _P, _L, _L, _F, _P],
    "p2hip_sample_snapshot": [_P, _P, _P, _P, _L, _P],
    "p2hip_cfr_iteration": [_P, _L, _I, _I, _P],
    "p2hip_write_scalars": [_P, _P, _P, _P, _P],
    "p2hip_stream_probe": [_P, _P, _L, _I, _I, _I, _P],
    "p2hip_placement_probe": [_P, _P, _L, _I, _P, _P],
    "p2hip_device_reserve": [_L, _P],
    "p2hip_device_release": [_P],
}
_RESTYPE = {"p2hip_error_string": ctypes.c_char_p, "p2hip_showdown_table_bytes": _L,
            "p2hip_tree_node_columns": _L}


class P2HipError(RuntimeError):
    pass


def library_path() -> str:
    return LIB_PATH


def load() -> ctypes.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise P2HipError(
                f"{LIB_PATH} is missing: build it with `python -m poker2_amd.build` "
                "(there is no fallback path)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _RESTYPE.get(name, _I)
        _lib = lib
    return _lib


def declared_symbols() -> list[str]:
    return list(_SIGNATURES)


def hip_is_available() -> bool:
    """True when the library loads and a GPU is visible to torch."""
    try:
        load()
    except (P2HipError, OSError):
        return False
    return torch.cuda.is_available()


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().p2hip_error_string(code)
        raise P2HipError(f"{what} failed: hip error {code} ({msg.decode() if msg else '?'})")


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def require_gpu(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        raise ValueError(f"{name} requires a GPU tensor (got device {t.device}).")


def call(name: str, *args) -> None:
    lib = load()
    check(getattr(lib, name)(*args), name)
