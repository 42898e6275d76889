"""The synthetic-input generator: Philox4x32-10 known answers and stream layout."""
import numpy as np

from gradhip import synth


def _kat(ctr, key):
    return [int(x) for x in synth.philox4x32(np.array([ctr], dtype=np.uint32), key)[0]]


def test_philox_known_answers():
    # Random123's published known-answer vectors for philox4x32-10.
    assert _kat([0, 0, 0, 0], (0, 0)) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert _kat([0xFFFFFFFF] * 4, (0xFFFFFFFF, 0xFFFFFFFF)) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6,
                                                                 0x6D5451FD]
    assert _kat([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], (0xA4093822, 0x299F31D0)) == [
        0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_streams_are_prefix_stable_and_distinct():
    a = synth.random_u32(1000, 7, 3)
    assert np.array_equal(a[:10], synth.random_u32(10, 7, 3))
    assert not np.array_equal(a[:10], synth.random_u32(10, 7, 4))
    assert not np.array_equal(a[:10], synth.random_u32(10, 8, 3))


def test_normal_moments_and_tokens_range():
    w = synth.normal(200_000, 1, 0, 0.02)
    assert w.dtype == np.float32
    assert abs(float(w.mean())) < 2e-4 and abs(float(w.std()) - 0.02) < 2e-4
    t = synth.uniform_tokens(50_000, 5000, 2)
    assert t.min() >= 0 and t.max() < 5000 and len(np.unique(t)) > 4900
    u = synth.uniforms(50_000, 3)
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(float(u.mean()) - 0.5) < 0.01


def test_preset_parameter_counts():
    # Counts grad.cpp's records give for the presets (BENCHMARKS.md:49-53; the
    # Modern count includes the 17 unused RMSNorm betas that stay in the file).
    def count(cfg):
        return sum(r * c for _, r, c, _ in synth.tensor_specs(cfg))
    c1, c2 = synth.PRESETS["c1"], synth.PRESETS["c2"]
    assert count(c2) == 68_961_792
    # the GPT-2 70M record is taken at the preset's own max_len of 1024
    c1_full = synth.Config(c1.arch, c1.vocab, c1.d_model, c1.layers, c1.heads, 1024)
    assert count(c1_full) == 69_778_944
    c0_full = synth.Config(synth.ARCH_GPT2, 5000, 512, 6, 8, 1024)
    assert count(c0_full) == 21_999_616
    assert c2.d_ff == 2048 and c1.d_ff == 3072
