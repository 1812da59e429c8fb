"""Givozen on the CPU: the engine's host logic (ragged scheduling, pages, passes of a loop on caches of their own,
checkpoint placement) with the package's torch restatement of the kernels, against the oracle."""
import pytest

from tests import _givozen as K
from tests import _givozen_cases as C

DEV = "cpu"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mechanisms(dtype):
    C.case_sandwich_norm(DEV, dtype)
    C.case_rotary_store(DEV, dtype)
    C.case_polynorm(DEV, dtype)
    C.case_moe_ff(DEV, dtype)


def test_inv_freq():
    C.case_inv_freq(DEV)


def test_moe_route_raw():
    C.case_moe_route_raw(DEV)


def test_router_logits():
    C.case_router_logits(DEV)


def test_attention_beacons():
    C.case_attention_beacons(DEV, "float32")


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


@pytest.mark.parametrize("seed", [102, 107])
def test_engine_random_configs(tmp_path, seed):
    C.case_engine_random_config(DEV, "float32", tmp_path, seed)


def test_engine_reuse_of_pages_and_slots(tmp_path):
    C.case_engine_reuse(DEV, "float32", tmp_path)


def test_engine_long_decode(tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate(tmp_path):
    C.case_generate(DEV, tmp_path)
