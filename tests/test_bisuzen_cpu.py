"""Bisuzen on the CPU: the engine's host logic (ragged scheduling, pages, state slots, passes of a loop on caches and
states of their own, checkpoint placement) with the package's torch restatement of the kernels, against the oracle."""
import pytest

from tests import _bisuzen as K
from tests import _bisuzen_cases as C

DEV = "cpu"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mechanisms(dtype):
    C.case_residual_dyt(DEV, dtype)
    C.case_qk_prep(DEV, dtype)
    C.case_glu_act(DEV, dtype)
    C.case_lightning(DEV, dtype)
    C.case_moe_ff(DEV, dtype)


def test_moe_route():
    C.case_moe_route(DEV)


def test_masked_attention():
    C.case_masked_attention(DEV, "float32")


def test_checkpoint_placement(tmp_path):
    C.case_checkpoint_placement(tmp_path)


def test_layer_by_layer(tmp_path):
    C.case_layer_by_layer(DEV, tmp_path)
    C.case_layer_by_layer(DEV, tmp_path / "odd", cfg=K.CFG_ODD)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_schedules(tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


@pytest.mark.parametrize("name", ["CFG_ODD", "CFG_WIDE", "CFG_ONE_PASS", "CFG_NO_LOOP"])
def test_engine_other_sizes(tmp_path, name):
    C.case_engine_schedules(DEV, "float32", tmp_path, cfg=getattr(K, name), seed=9)


@pytest.mark.parametrize("seed", [101, 104])
def test_engine_random_configs(tmp_path, seed):
    C.case_engine_random_config(DEV, "float32", tmp_path, seed)


def test_engine_long_windows(tmp_path):
    C.case_engine_long_windows(DEV, "float32", tmp_path)


def test_engine_reuse_of_pages_and_slots(tmp_path):
    C.case_engine_reuse(DEV, "float32", tmp_path)


def test_engine_long_decode(tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate(tmp_path):
    C.case_generate(DEV, tmp_path)
