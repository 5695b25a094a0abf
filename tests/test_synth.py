"""The synthetic-payload generator against a NumPy restatement of its specification."""
import numpy as np
import pytest

import np_blocks as nb

M64 = np.uint64


def mix(z):
    with np.errstate(over="ignore"):
        z = (z + M64(0x9E3779B97F4A7C15)).astype(np.uint64)
        z = ((z ^ (z >> M64(30))) * M64(0xBF58476D1CE4E5B9)).astype(np.uint64)
        z = ((z ^ (z >> M64(27))) * M64(0x94D049BB133111EB)).astype(np.uint64)
        return z ^ (z >> M64(31))


def key(seed, tid):
    return mix(np.array([seed], dtype=np.uint64) ^ mix(np.array([tid], dtype=np.uint64)))[0]


def words(seed, tid, b, n):
    with np.errstate(over="ignore"):
        return mix(key(seed, tid) + M64(32) * M64(b) + np.arange(n, dtype=np.uint64))


def scale(lo, hi, r):
    u = float(int(r) & 0xFFFFFF) / 16777216.0
    return np.frombuffer(np.float16(np.float32(lo + (hi - lo) * u)).tobytes(), dtype=np.uint8)


def ref_block(t, seed, tid, b, lo, hi):
    if t == 8:
        w = words(seed, tid, b, 9)
        v = w[1:].view(np.uint16).astype(np.uint32)          # little-endian: 4 x u16 per word, low first
        q = ((v * 255) >> 16).astype(np.int32) - 127
        return np.concatenate([scale(lo, hi, w[0]), q.astype(np.int8).view(np.uint8)])
    if t == 2:
        w = words(seed, tid, b, 3)
        return np.concatenate([scale(lo, hi, w[0]), w[1:].view(np.uint8)])
    if t == 3:
        w = words(seed, tid, b, 3)
        return np.concatenate([scale(lo, hi, w[0]), scale(-8.0 * lo, -8.0 * hi, int(w[0]) >> 32), w[1:].view(np.uint8)])
    if t == 6:
        w = words(seed, tid, b, 3)
        return np.concatenate([scale(lo, hi, w[0]), w[0:1].view(np.uint8)[4:], w[1:].view(np.uint8)])
    if t == 7:
        w = words(seed, tid, b, 4)
        return np.concatenate([scale(lo, hi, w[0]), scale(-16.0 * lo, -16.0 * hi, int(w[0]) >> 32), w[3:4].view(np.uint8)[:4], w[1:3].view(np.uint8)])
    if t == 10:
        w = words(seed, tid, b, 11)
        return np.concatenate([w[:10].view(np.uint8), scale(lo, hi, w[10]), scale(lo, hi, int(w[10]) >> 32)])
    if t == 11:
        w = words(seed, tid, b, 15)
        return np.concatenate([w[:13].view(np.uint8), w[13:14].view(np.uint8)[:4], scale(lo, hi, w[14])])
    if t == 12:
        w = words(seed, tid, b, 19)
        sc = w[1:2].view(np.uint8) & 63
        mn = w[2:3].view(np.uint8) & 63
        return np.concatenate([scale(lo, hi, w[0]), scale(lo, hi, int(w[0]) >> 32), nb.pack_q4k_scales(sc, mn), w[3:].view(np.uint8)])
    if t == 13:
        w = words(seed, tid, b, 23)
        sc = w[1:2].view(np.uint8) & 63
        mn = w[2:3].view(np.uint8) & 63
        return np.concatenate([scale(lo, hi, w[0]), scale(lo, hi, int(w[0]) >> 32), nb.pack_q4k_scales(sc, mn), w[3:].view(np.uint8)])
    w = words(seed, tid, b, 27)
    sc = ((w[24:26].view(np.uint8) & 63).astype(np.int32) - 32).astype(np.int8).view(np.uint8)
    return np.concatenate([w[:24].view(np.uint8), sc, scale(lo, hi, w[26])])


@pytest.mark.parametrize("t", [8, 2, 3, 6, 7, 10, 11, 12, 13, 14])
def test_blocks_follow_the_specification(lib, t):
    from rustorch_amd import synth, GGMLType
    lo, hi = synth.D_RANGE[GGMLType(t)]
    be, bb = GGMLType(t).block_elems(), GGMLType(t).type_size()
    raw = synth.blocks(t, 42, 7, 5, 2 * be).reshape(-1, bb)
    for b in (0, 1, 9):
        assert np.array_equal(raw[b], ref_block(t, 42, 7, b, lo, hi)), (t, b)
    # a tensor is a pure function of (seed, tensor_id): prefix property and sensitivity
    assert np.array_equal(synth.blocks(t, 42, 7, 2, 2 * be).reshape(-1, bb), raw[:4])
    assert not np.array_equal(synth.blocks(t, 43, 7, 5, 2 * be).reshape(-1, bb), raw)
    assert not np.array_equal(synth.blocks(t, 42, 8, 5, 2 * be).reshape(-1, bb), raw)


def test_field_ranges_of_the_configurations(lib):
    from rustorch_amd import synth
    n = 512
    raw = synth.blocks(8, 1, 1, n, 32).reshape(n, 34)
    d = raw[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    q = raw[:, 2:].view(np.int8)
    assert d.min() >= 1e-4 * 0.999 and d.max() <= 2e-3 * 1.001 and q.min() == -127 and q.max() == 127
    raw = synth.blocks(2, 1, 1, n, 32).reshape(n, 18)
    d = raw[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    assert d.min() >= 1e-3 * 0.999 and d.max() <= 2e-2 * 1.001
    assert set(np.unique(raw[:, 2:] & 15)) == set(range(16)) and set(np.unique(raw[:, 2:] >> 4)) == set(range(16))
    raw = synth.blocks(12, 1, 1, n, 256).reshape(n, 144)
    dd = raw[:, :4].copy().view(np.float16).astype(np.float32)
    assert dd.min() >= 1e-3 * 0.999 and dd.max() <= 1e-2 * 1.001
    scm = np.array([[nb.q4k_scale_min(r[4:16], j) for j in range(8)] for r in raw[:64]])
    assert scm.min() == 0 and scm.max() == 63
    raw = synth.blocks(14, 1, 1, n, 256).reshape(n, 210)
    sc = raw[:, 192:208].view(np.int8)
    d = raw[:, 208:210].copy().view(np.float16).astype(np.float32)
    assert sc.min() == -32 and sc.max() == 31 and d.min() >= 1e-3 * 0.999 and d.max() <= 1e-2 * 1.001


def test_normal_and_tokens(lib):
    from rustorch_amd import synth
    x = synth.normal(3, 5, 200001)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01 and np.isfinite(x).all()
    assert np.array_equal(synth.normal(3, 5, 1000), x[:1000])
    g = synth.normal(3, 6, 100000, 1.0, 0.01)
    assert abs(g.mean() - 1) < 1e-3 and abs(g.std() - 0.01) < 1e-3
    t = synth.tokens(3, 4, 5000, 32000)
    assert t.min() >= 0 and t.max() < 32000 and len(np.unique(t)) > 4000


def test_config_weight_bytes(lib):
    # the per-layer and per-model byte counts the bench prices bandwidth against
    from rustorch_amd import synth, GGMLType
    assert synth.layer_weight_bytes(4096, 11008) == 129_785_856
    assert GGMLType.Q8_0.row_bytes(4096) * 4096 == 17_825_792
    assert GGMLType.Q4_0.row_bytes(4096) * 11008 == 25_362_432 == GGMLType.Q4_0.row_bytes(11008) * 4096
    assert 32 * 129_785_856 + GGMLType.Q6_K.row_bytes(4096) * 32000 == 4_260_667_392
