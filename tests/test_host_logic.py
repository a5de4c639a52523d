"""Host-side logic of the product that needs no GPU: parameter arithmetic, file formats, datasets."""
import numpy as np

from glide_amd import datasets as D
from glide_amd import index as G
from oracle import oracle as O


def test_parameter_arithmetic_matches_reference_restatement():
    for beam in (1, 31, 32, 33, 50, 64, 100, 128, 200, 256, 300, 512):
        for degree in (16, 32, 64, 96, 128, 256):
            mi, b = G.adjust_search_params(0, 0, beam)
            assert (mi, b) == O.adjust_search_params(0, 0, beam)
            hb = G.calculate_hash_bitlen(b, degree, 0.5, 0)
            assert hb == O.hash_bitlen(b, degree, 0.5, 0)
            assert G.calculate_hash_reset_interval(b, degree, 0.5, hb) == O.hash_reset_interval(b, degree, 0.5, hb)
    assert G.adjust_search_params(90, 0, 64) == O.adjust_search_params(90, 0, 64)
    assert G.adjust_search_params(0, 500, 70) == O.adjust_search_params(0, 500, 70)
    p = G.make_search_parameter(50, 32)
    assert (p.beam, p.max_iterations, p.hash_bit, p.hash_reset_interval) == (64, 56, 8, 2)   # test.sh search beam 50
    assert G.NNDescentParameter(graph_degree=32).intermediate_graph_degree == 48


def test_unsupported_sizes_raise_like_the_reference():
    import pytest
    with pytest.raises(ValueError, match="Unsupported beam"):
        G._check_sizes(513, 32)
    with pytest.raises(ValueError, match="Unsupported beam"):
        G._check_sizes(300, 32)        # above 256 a beam is a multiple of 16; adjust_search_params never hands out another
    for beam in (1, 50, 255, 256, 288, 320, 448, 480, 512):
        G._check_sizes(beam, 32)
    assert all(G.adjust_search_params(0, 0, b)[1] % 32 == 0 for b in range(1, 513))
    with pytest.raises(ValueError, match="Unsupported graph_degree"):
        G._check_sizes(64, 257)


def test_file_formats_round_trip(tmp_path):
    rng = np.random.default_rng(0)
    m = rng.standard_normal((7, 5)).astype(np.float32)
    D.write_fbin(tmp_path / "m.fbin", m)
    raw = np.fromfile(tmp_path / "m.fbin", dtype=np.uint32)
    assert raw[0] == 7 and raw[1] == 5 and raw.size == 2 + 35           # u32 num, u32 dim, rows
    assert np.array_equal(D.read_fbin(tmp_path / "m.fbin"), m)
    g = rng.integers(0, 100, (4, 3)).astype(np.uint32)
    D.write_fbin(tmp_path / "g", g)
    assert np.array_equal(D.read_fbin(tmp_path / "g", np.uint32), g)
    D.write_vector(tmp_path / "v", [3, 1, 4])
    assert np.fromfile(tmp_path / "v", dtype=np.uint32).tolist() == [3, 3, 1, 4]
    assert D.read_vector(tmp_path / "v").tolist() == [3, 1, 4]
    D.write_segment(tmp_path / "s", [0, 10, 30], [10, 20, 5])
    assert np.fromfile(tmp_path / "s", dtype=np.uint32).tolist() == [3, 0, 10, 30, 10, 20, 5]   # n, starts, lengths
    s, l = D.read_segment(tmp_path / "s")
    assert s.tolist() == [0, 10, 30] and l.tolist() == [10, 20, 5]


def test_synthetic_generators_are_seeded_and_shaped():
    a, b = D.gmm_clipped(1000, 128, seed=5), D.gmm_clipped(1000, 128, seed=5)
    assert np.array_equal(a, b) and a.dtype == np.float32
    assert a.min() >= 0 and a.max() <= 255 and np.array_equal(a, np.rint(a))
    assert not np.array_equal(a, D.gmm_clipped(1000, 128, seed=6))
    c = D.gmm_normalized(500, 96)
    assert np.allclose(np.linalg.norm(c, axis=1), 1, atol=1e-5)
    e = D.beta_scaled(200, 960)
    assert e.shape == (200, 960) and e.min() >= 0 and e.max() <= 1
    r = D.recall(np.array([[1, 2, 3]]), np.array([[3, 4, 1]]), 3)
    assert abs(r - 2 / 3) < 1e-9
