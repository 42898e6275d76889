"""The C-ABI boundary: the library loads without a GPU, exports exactly what
include/gradhip.h declares, and refuses to compute without a device."""
import os
import re

import numpy as np
import pytest

import gradhip as G
from gradhip import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "gradhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gh_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_name_the_same_symbols():
    names = _declared()
    assert len(names) >= 20
    assert names == sorted(G.SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = G.load_library()
    for name in _declared():
        assert getattr(lib, name) is not None


def test_header_cites_the_reference_for_every_entry_point():
    text = open(os.path.join(ROOT, "include", "gradhip.h")).read()
    for cite in ("inference.cpp:150-258", "inference.cpp:121-148", "gpt_model.cpp:383-525",
                 "gpt_model.cpp:292-381", "text_gen.cpp:37-91", "text_gen.cpp:135-209",
                 "text_gen.cpp:14-33", "inference.h:20-22"):
        assert cite in text


def test_struct_layouts_match_the_header():
    import ctypes as C
    assert C.sizeof(G.GhConfig) == 48 and G.GhConfig.tokenizer_hash.offset == 40
    assert C.sizeof(G.GhSessionOpts) == 20
    assert C.sizeof(G.GhSampling) == 20
    assert C.sizeof(G.GhTiming) == 24 and G.GhTiming.row_picks.offset == 20


def test_host_logic_runs_without_a_gpu():
    cfg = synth.Config(synth.ARCH_MODERN, 11, 8, 2, 2, 6)
    c = G._cfg_struct(cfg)
    lib = G.load_library()
    import ctypes as C
    assert lib.gh_config_num_tensors(C.byref(c)) == len(synth.tensor_specs(cfg))
    r, k = C.c_int32(), C.c_int32()
    for i, (_, rows, cols, _) in enumerate(synth.tensor_specs(cfg)):
        assert lib.gh_config_tensor_shape(C.byref(c), i, C.byref(r), C.byref(k)) == G.GH_OK
        assert (r.value, k.value) == (rows, cols)
    assert lib.gh_config_tensor_shape(C.byref(c), 999, C.byref(r), C.byref(k)) == G.GH_ERR_OUT_OF_RANGE
    bad = G._cfg_struct(synth.Config(synth.ARCH_MODERN, 11, 9, 1, 3, 6))
    assert lib.gh_config_num_tensors(C.byref(bad)) == -1
    assert b"RoPE requires an even head size" in lib.gh_last_error()


def _has_gpu():
    try:
        G.device_info()
        return True
    except G.DeviceError:
        return False


@pytest.mark.skipif(_has_gpu(), reason="checks the no-GPU failure mode")
def test_compute_fails_loudly_without_a_gpu(tmp_path):
    cfg = synth.Config(synth.ARCH_GPT2, 11, 8, 1, 2, 6)
    W = synth.make_weights(cfg, 1)
    with pytest.raises(G.DeviceError, match="no CPU fallback"):
        G.Model.from_tensors(cfg, W)
    path = str(tmp_path / "m.bin")
    synth.write_checkpoint(path, cfg, W)
    with pytest.raises(G.DeviceError, match="no CPU fallback"):
        G.Model.load(path)
