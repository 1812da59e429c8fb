"""liblvmix.so loads without a GPU, exports exactly what include/lv_mixers.h declares with the argument counts the
ctypes table binds, and rejects bad arguments on the host before any launch."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lv_mixers.h")


def declared():
    """name -> number of parameters of every function the header declares."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"\b(lv_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = args.strip()
        out[name] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def test_header_and_ctypes_table_agree():
    from light_vllm_amd import _mixlib
    decl = declared()
    assert sorted(decl) == sorted(_mixlib.SIGNATURES)
    for name, (_, args) in _mixlib.SIGNATURES.items():
        assert len(args) == decl[name], name
    lib = _mixlib.load()
    for name in decl:
        assert hasattr(lib, name), f"{name} missing from liblvmix.so"
    assert lib.lv_mix_abi_version() == _mixlib.ABI_VERSION
    version = int(re.search(r"#define LV_MIX_ABI_VERSION (\d+)", open(HEADER).read()).group(1))
    assert version == _mixlib.ABI_VERSION


def test_argument_validation_happens_before_any_launch():
    from light_vllm_amd import _mixlib
    lib = _mixlib.load()
    buf = ctypes.create_string_buffer(256)
    p = (ctypes.addressof(buf) + 15) & ~15
    # zero tokens: nothing to do, whatever else is passed
    assert lib.lv_sandwich_add_norm(None, None, None, None, None, None, 1.0, None, 0, 64, 1e-6, 0, None) == 0
    assert lib.lv_rotary_store(None, 0, 0, 0, 0, None, None, None, None, None, None, None, None, None, 1, 0, 4, 2, 8, 8, 4, 16, 0, None) == 0
    assert lib.lv_polynorm(None, 0, None, None, 0, 8, 1e-6, 0, None) == 0
    assert lib.lv_expert_glu(None, 0, None, None, 0, None, 0, 0, 2, 8, 1.0, 1.702, 0, None) == 0
    # a sublayer output without its norm weight; an output without a norm weight
    assert lib.lv_sandwich_add_norm(p, p, None, None, None, p, 1.0, p, 1, 8, 1e-6, 0, None) == -1
    assert lib.lv_sandwich_add_norm(p, None, None, None, None, None, 1.0, p, 1, 8, 1e-6, 0, None) == -1
    assert lib.lv_sandwich_add_norm(p, None, None, None, None, p, 1.0, p, 1, 1 << 20, 1e-6, 0, None) == -2     # row above the LDS
    # an odd number of rotated entries, more of them than the head has, heads that do not divide, columns past the row
    args = lambda **kw: [p, kw.get("ld", 64), 0, 32, 48, p, None, p, p, p, p, p, p, p, 1, 1, kw.get("H", 4), kw.get("G", 2), 8, 8,  # noqa: E731
                         kw.get("rot", 4), 16, 0, None]
    assert lib.lv_rotary_store(*args(rot=3)) == -1
    assert lib.lv_rotary_store(*args(rot=10)) == -1
    assert lib.lv_rotary_store(*args(H=3)) == -1
    assert lib.lv_rotary_store(*args(ld=40)) == -1 and b"lv_rotary_store" in lib.lv_mix_last_error()
    assert lib.lv_polynorm(p, 4, p, p, 1, 8, 1e-6, 0, None) == -1                      # row stride below the row
    assert lib.lv_polynorm(p, 8, p, p, 1, 8, 1e-6, 7, None) == -1                      # unknown dtype
    assert lib.lv_expert_glu(p, 8, None, None, 0, p, 8, 1, 2, 8, 1.0, 1.702, 0, None) == -1     # two experts need 32 columns
    assert lib.lv_moe_route(p, None, p, p, None, 1, 4, 5, 1, 1, 0, None) == -1                 # more choices than experts
    assert lib.lv_router_logits(p, 4, p, p, 1, 8, 4, 0, None) == -1                            # row stride below the row
    assert lib.lv_moe_grouped_glu_ff(p, p, p, p, p, 0, p, p, 1, 48, 32, 4, 2, 1.0, 1.702, None) == -1     # width no multiple of 32
    assert lib.lv_moe_grouped_glu_ff(p, p, p, p, p, 100, p, p, 1, 64, 32, 4, 2, 1.0, 1.702, None) == -1   # down rows shorter than E*F
    assert lib.lv_window_pool_attn(p, p, p, None, None, p, 4, p, p, p, p, p, 1, 1, 4, 2, 8, 8, 16, 64, 0, 0.5, 0, 0, 0, 5, 0, None) == -1   # gate kind
