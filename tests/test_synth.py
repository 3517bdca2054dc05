"""The synthetic generators are counter based: any slice equals the same slice
of the whole stream, whatever the chunking."""
import numpy as np

from coral_amd import synth


def test_streams_are_sliceable():
    whole = synth.normal(77, 0, 1001)
    for s, c in ((0, 1), (1, 1), (3, 10), (500, 501), (999, 2)):
        assert np.array_equal(synth.normal(77, s, c), whole[s:s + c])
    u = synth.uniform01(5, 0, 100)
    assert np.array_equal(synth.uniform01(5, 40, 7), u[40:47])
    assert (u > 0).all() and (u < 1).all()


def test_splitmix64_known_answer():
    # first outputs of the published SplitMix64 for seed 0 (state advances by the golden gamma)
    out = synth.splitmix64(0, np.arange(3, dtype=np.uint64))
    assert [int(x) for x in out] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]


def test_matrix_rows_do_not_depend_on_chunking():
    a = synth.gaussian_matrix(9, 100, 12, chunk_rows=7)
    b = synth.gaussian_matrix(9, 100, 12, chunk_rows=1000)
    assert np.array_equal(a, b)
    assert np.array_equal(synth.gaussian_matrix(9, 10, 12, row0=40), a[40:50])
    assert abs(a.mean()) < 0.1 and abs(a.std() - 1) < 0.1


def test_query_laws():
    q = synth.shifted_queries(2000, 16, 1, 2, 3)
    s = q.std(axis=0)
    assert q.shape == (2000, 16) and s.min() > 0.4 and s.max() < 1.6 and s.max() - s.min() > 0.3
    c = synth.cone_queries(500, 32, 4, 5)
    assert np.allclose(np.linalg.norm(c, axis=1), 1, atol=1e-5)
    assert (c @ c.mean(0)).min() > 0  # all inside one cone


def test_tombstones_and_graph():
    m = synth.tombstone_mask(1000, 5002)
    bits = np.unpackbits(m.view(np.uint8), bitorder="little")[:1000]
    ids = np.arange(1000, dtype=np.uint64)
    assert np.array_equal(bits.astype(bool), synth.splitmix64(5002, ids) % np.uint64(10) == 0)
    assert 50 < bits.sum() < 150
    base = synth.gaussian_matrix(1, 300, 8)
    g = synth.exact_knn_graph(base, 5, block=64)
    d = ((base[:, None, :].astype(np.float64) - base[None, :, :]) ** 2).sum(-1)
    np.fill_diagonal(d, np.inf)
    assert np.array_equal(g, np.argsort(d, axis=1, kind="stable")[:, :5].astype(np.int32))
    assert synth.medoid_start(base) == int(np.argmin(((base - base.mean(0)) ** 2).sum(1)))
