"""Pins the oracle's pack/unpack: memcpy at running offsets
(ops/collective_operations.cc:68-112) and the 16-byte padded GPU layout
(ops/gpu_operations.cc:127-153,238-275)."""
import numpy as np

SIZES = [0, 1, 2, 3, 15, 16, 17, 31, 32, 33, 100, 4095, 4096, 4097]


def _tensors(rng, sizes):
    return [rng.integers(0, 256, n, dtype=np.uint8) for n in sizes]


def test_pack_is_concatenation(orc):
    rng = np.random.default_rng(0)
    ts = _tensors(rng, SIZES)
    buf, n = orc.pack(ts)
    assert n == sum(SIZES)
    assert np.array_equal(buf[:n], np.concatenate(ts))
    assert np.all(buf[n:] == 0xAB)  # nothing written past buffer_len


def test_pack_brute_force_byte_map(orc):
    # tensor i is filled with byte i+1: every buffer byte names its source tensor
    ts = [np.full(n, i + 1, np.uint8) for i, n in enumerate(SIZES)]
    buf, n = orc.pack(ts)
    off = 0
    for i, sz in enumerate(SIZES):
        assert np.all(buf[off:off + sz] == i + 1)
        off += sz
    assert off == n


def test_unpack_round_trip(orc):
    rng = np.random.default_rng(1)
    ts = _tensors(rng, SIZES)
    buf, n = orc.pack(ts)
    outs = [np.zeros_like(t) for t in ts]
    orc.unpack(buf, outs)
    for t, o in zip(ts, outs):
        assert np.array_equal(t, o)


def test_padded_offsets_closed_form(orc):
    offs = orc.padded_offsets(SIZES)
    want = np.concatenate([[0], np.cumsum([16 * ((s + 15) // 16) for s in SIZES])])
    assert np.array_equal(offs, want)
    assert all(o % 16 == 0 for o in offs)


def test_padded_pack_places_each_tensor_at_its_offset(orc):
    ts = [np.full(n, i + 1, np.uint8) for i, n in enumerate(SIZES)]
    buf, n = orc.pack(ts, padded=True)
    offs = orc.padded_offsets(SIZES)
    assert n == offs[-1]
    for i, sz in enumerate(SIZES):
        assert np.all(buf[offs[i]:offs[i] + sz] == i + 1)
        assert np.all(buf[offs[i] + sz:offs[i + 1]] == 0xAB)  # pad bytes untouched by the reference
    outs = [np.zeros_like(t) for t in ts]
    orc.unpack(buf, outs, padded=True)
    for t, o in zip(ts, outs):
        assert np.array_equal(t, o)


def test_empty_entry_list(orc):
    buf, n = orc.pack([])
    assert n == 0
