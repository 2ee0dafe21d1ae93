"""Pins the oracle's pack / unpack / transposing pack / bf16->fp8 against
independent models: per-byte numpy indexing, numpy transpose, torch's
float8_e4m3fn cast."""
import ctypes as C

import numpy as np
import pytest

import checkers


def _random_runs(rng, cap, n, max_len=300):
    """n non-overlapping (in dst) ranges inside [0, cap)"""
    runs, used = [], np.zeros(cap, dtype=bool)
    tries = 0
    while len(runs) < n and tries < 10000:
        tries += 1
        ln = int(rng.integers(1, max_len))
        s = int(rng.integers(0, cap - ln))
        d = int(rng.integers(0, cap - ln))
        if used[d:d + ln].any():
            continue
        used[d:d + ln] = True
        runs.append((s, d, ln))
    return np.array(runs, dtype=np.uint64)


@pytest.mark.parametrize("seed", range(5))
def test_pack_is_concatenation_of_source_ranges(seed):
    rng = np.random.default_rng(seed)
    layer = rng.integers(0, 256, size=20000, dtype=np.uint8)
    runs = _random_runs(rng, len(layer), 60)
    blob = checkers.oracle_pack(layer, runs)
    expect = np.concatenate([layer[int(s):int(s + n)] for s, _, n in runs])
    assert np.array_equal(blob, expect)
    # byte-at-a-time model
    k = 0
    for s, _, n in runs[:10]:
        for j in range(int(n)):
            assert blob[k + j] == layer[int(s) + j]
        k += int(n)


@pytest.mark.parametrize("seed", range(5))
def test_unpack_scatters_and_touches_nothing_else(seed):
    rng = np.random.default_rng(100 + seed)
    src = rng.integers(0, 256, size=20000, dtype=np.uint8)
    runs = _random_runs(rng, len(src), 60)
    blob = checkers.oracle_pack(src, runs)
    dst = rng.integers(0, 256, size=20000, dtype=np.uint8)
    before = dst.copy()
    checkers.oracle_unpack(dst, runs, blob)
    touched = np.zeros(len(dst), dtype=bool)
    for s, d, n in runs:
        s, d, n = int(s), int(d), int(n)
        assert np.array_equal(dst[d:d + n], src[s:s + n])
        touched[d:d + n] = True
    assert np.array_equal(dst[~touched], before[~touched])


def test_pack_layers_threads_agree_with_single_thread():
    rng = np.random.default_rng(7)
    lib = checkers.oracle()
    layers = [rng.integers(0, 256, size=5000, dtype=np.uint8) for _ in range(6)]
    runs = _random_runs(rng, 5000, 20)
    total = int(runs[:, 2].sum())
    ptrs = (C.c_void_p * 6)(*[l.ctypes.data for l in layers])
    a = np.zeros(6 * total, dtype=np.uint8)
    b = np.zeros(6 * total, dtype=np.uint8)
    lib.kvto_pack_layers(ptrs, 6, runs.ctypes.data, len(runs), a.ctypes.data, total, 1)
    lib.kvto_pack_layers(ptrs, 6, runs.ctypes.data, len(runs), b.ctypes.data, total, 4)
    assert np.array_equal(a, b)
    for i, l in enumerate(layers):
        assert np.array_equal(a[i * total:(i + 1) * total], checkers.oracle_pack(l, runs))
    outs = [np.zeros(5000, dtype=np.uint8) for _ in range(6)]
    optrs = (C.c_void_p * 6)(*[o.ctypes.data for o in outs])
    lib.kvto_unpack_layers(optrs, 6, runs.ctypes.data, len(runs), a.ctypes.data, total, 3)
    for l, o in zip(layers, outs):
        ref = np.zeros(5000, dtype=np.uint8)
        checkers.oracle_unpack(ref, runs, checkers.oracle_pack(l, runs))
        assert np.array_equal(o, ref)


@pytest.mark.parametrize("heads,ntpb,row", [(2, 3, 4), (8, 16, 256), (4, 16, 64), (1, 5, 16)])
def test_transposing_pack_is_the_textbook_permutation(heads, ntpb, row):
    rng = np.random.default_rng(heads * 100 + ntpb)
    lib = checkers.oracle()
    nblk = 7
    cache = rng.integers(0, 256, size=(nblk, 2, heads, ntpb, row), dtype=np.uint8)
    ids = np.array([5, 0, 3], dtype=np.uint32)
    blob = np.zeros((3, 2, ntpb, heads, row), dtype=np.uint8)
    lib.kvto_pack_hnd_to_nhd(cache.ctypes.data, ids.ctypes.data, 3, heads, ntpb, row,
                             blob.ctypes.data)
    assert np.array_equal(blob, cache[ids].transpose(0, 1, 3, 2, 4))
    # equals a plain pack of the NHD cache that holds the same logical values
    nhd = np.ascontiguousarray(cache.transpose(0, 1, 3, 2, 4))
    B = 2 * heads * ntpb * row
    runs = np.array([(int(i) * B, 0, B) for i in ids], dtype=np.uint64)
    assert np.array_equal(blob.reshape(-1), checkers.oracle_pack(nhd.reshape(-1), runs))
    # round trip
    back = np.zeros_like(cache)
    lib.kvto_unpack_nhd_to_hnd(back.ctypes.data, ids.ctypes.data, 3, heads, ntpb, row,
                               blob.ctypes.data)
    assert np.array_equal(back[ids], cache[ids])
    rest = np.setdiff1d(np.arange(nblk), ids)
    assert not back[rest].any()


def test_bf16_to_fp8_all_bit_patterns_against_torch():
    torch = pytest.importorskip("torch")
    lib = checkers.oracle()
    bits = np.arange(65536, dtype=np.uint16)
    got = np.array([lib.kvto_bf16_to_fp8(int(b)) for b in bits], dtype=np.uint8)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    finite = torch.isfinite(x) & (x.float().abs() <= 448.0)
    ref = x.float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    f = finite.numpy()
    assert np.array_equal(got[f], ref[f])
    # beyond the finite range: saturate to +-448 (0x7E); NaN stays NaN (0x7F)
    xf = x.float()
    big = (torch.isinf(xf) | (xf.abs() > 448.0)).numpy() & ~torch.isnan(xf).numpy()
    # values in (448, 464) still round down to 448 under RNE; all map to 0x7E either way
    assert np.all((got[big] & 0x7F) == 0x7E)
    assert np.all((got[big] >> 7) == (bits[big] >> 15))
    nan = torch.isnan(xf).numpy()
    assert np.all((got[nan] & 0x7F) == 0x7F)


def test_converting_pack_halves_the_bytes():
    torch = pytest.importorskip("torch")
    lib = checkers.oracle()
    g = torch.Generator().manual_seed(3)
    vals = (torch.rand(4096, generator=g) * 2 - 1).to(torch.bfloat16)
    layer = vals.view(torch.int16).numpy().view(np.uint8)
    # lengths are fp8 byte counts; sources are bf16 (2 bytes per element)
    runs = np.array([(512, 0, 100), (4096, 100, 256)], dtype=np.uint64)
    blob = np.zeros(356, dtype=np.uint8)
    lib.kvto_pack_bf16_to_fp8(layer.ctypes.data, runs.ctypes.data, 2, blob.ctypes.data)
    e0 = vals[256:356].float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    e1 = vals[2048:2304].float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(blob, np.concatenate([e0, e1]))
