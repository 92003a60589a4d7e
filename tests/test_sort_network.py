"""The index kernel folds a lane's queue into its list with a fixed compare-exchange network; a network sorts every
input iff it sorts every zero-one input (Knuth, TAOCP 3, 5.3.4), so all 2^13 of them are tried here on the comparator
table as it stands in the kernel's source."""
import pathlib
import re

import numpy as np

SRC = pathlib.Path(__file__).resolve().parents[1] / "speed3r_amd" / "csrc" / "compressed_mfma.hip"


def _table():
    text = SRC.read_text()
    size = int(re.search(r"kSortNet13Size\s*=\s*(\d+);", text).group(1))
    body = re.search(r"kSortNet13\[kSortNet13Size\]\[2\]\s*=\s*\{(.*?)\};", text, re.S).group(1)
    pairs = [(int(a), int(b)) for a, b in re.findall(r"\{(\d+),\s*(\d+)\}", body)]
    assert len(pairs) == size
    return pairs


def _run(pairs, x):  # x: [cases, 13]; a comparator (i, j) leaves the larger value at i (descending order)
    x = x.copy()
    for i, j in pairs:
        hi, lo = np.maximum(x[:, i], x[:, j]), np.minimum(x[:, i], x[:, j])
        x[:, i], x[:, j] = hi, lo
    return x


def test_network_sorts_every_zero_one_input():
    pairs = _table()
    assert all(0 <= i < j < 13 for i, j in pairs)
    bits = ((np.arange(1 << 13)[:, None] >> np.arange(13)[None, :]) & 1).astype(np.int8)
    out = _run(pairs, bits)
    assert (out[:, :-1] >= out[:, 1:]).all()
    assert (out.sum(1) == bits.sum(1)).all()


def test_network_sorts_random_keys_with_ties():
    pairs = _table()
    rng = np.random.default_rng(0)
    x = rng.integers(0, 6, size=(4096, 13)).astype(np.float64)  # many equal keys
    out = _run(pairs, x)
    assert np.array_equal(out, -np.sort(-x, axis=1))


def test_a_broken_network_is_caught():
    pairs = _table()
    bits = ((np.arange(1 << 13)[:, None] >> np.arange(13)[None, :]) & 1).astype(np.int8)
    for drop in (0, len(pairs) // 2, len(pairs) - 1):
        out = _run(pairs[:drop] + pairs[drop + 1:], bits)
        assert not (out[:, :-1] >= out[:, 1:]).all()
