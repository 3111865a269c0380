"""C oracle against the committed golden fixtures (tests/golden/) and the Philox pins. CPU only."""
import numpy as np
import pytest

from golden_util import (BMM_CASES, CONV_CASES, PACK_WIDTHS, POOL_CASES, SMP_CASES, TAGS, load_ops, load_philox)

G = load_ops()


@pytest.mark.parametrize("tag", TAGS)
def test_pack(oracle, tag):
    for C in PACK_WIDTHS:
        np.testing.assert_array_equal(oracle.pack(G[f"pack_{tag}_C{C}_in"], TAGS[tag]), G[f"pack_{tag}_C{C}_out"])
        un = oracle.unpack(G[f"pack_{tag}_C{C}_out"])
        np.testing.assert_array_equal(un[:, :C], G[f"pack_{tag}_C{C}_in"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", BMM_CASES)
def test_bmm(oracle, tag, case):
    A, B = G[f"bmm_{tag}_{case}_A"], G[f"bmm_{tag}_{case}_B"]
    np.testing.assert_array_equal(oracle.bmm(A, B), G[f"bmm_{tag}_{case}_C"])
    np.testing.assert_array_equal(oracle.bmm_act(A, B, G[f"bmm_{tag}_{case}_thr"]), G[f"bmm_{tag}_{case}_act"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv(oracle, tag, case):
    x, f = G[f"conv_{tag}_{case}_x"], G[f"conv_{tag}_{case}_f"]
    geom = [int(v) for v in G[f"conv_{tag}_{case}_geom"]]
    np.testing.assert_array_equal(oracle.batch_im2col(x, *geom), G[f"conv_{tag}_{case}_cols"])
    np.testing.assert_array_equal(oracle.conv(x, f, *geom), G[f"conv_{tag}_{case}_popc"])
    np.testing.assert_array_equal(oracle.conv_act(x, f, G[f"conv_{tag}_{case}_thr"], *geom),
                                  G[f"conv_{tag}_{case}_act"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", POOL_CASES)
def test_pool(oracle, tag, case):
    geom = [int(v) for v in G[f"pool_{tag}_{case}_geom"]]
    np.testing.assert_array_equal(oracle.max_pool2d(G[f"pool_{tag}_{case}_x"], *geom), G[f"pool_{tag}_{case}_out"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", SMP_CASES)
def test_sampling(oracle, tag, case):
    p = f"smp_{tag}_{case}_"
    words, thr, base, x = G[p + "words"], G[p + "thr"], G[p + "base"], G[p + "x"]
    T = 214748364
    np.testing.assert_array_equal(oracle.sample_from_words(thr, words, TAGS[tag]), G[p + "sample"])
    np.testing.assert_array_equal(oracle.sample_from_words(T, words, TAGS[tag], base=base), G[p + "flip"])
    np.testing.assert_array_equal(oracle.seeded_bmv_from_words(thr, x, words), G[p + "bmv_sample"])
    np.testing.assert_array_equal(oracle.seeded_bmv_from_words(T, x, words, base=base), G[p + "bmv_flip"])


def test_philox_known_answers(oracle):
    P = load_philox()
    for kat in P["random123_kat"]:
        assert [int(v) for v in oracle.philox4x32_10(kat["ctr"], kat["key"])] == kat["out"]
    for case in P["rocrand"]:
        got = oracle.philox_words(case["seed"], case["subsequence"], case["offset"], len(case["words"]))
        assert [int(v) for v in got] == case["words"]
