"""The synthetic workload generator: the numpy streams and their torch twins (which the GPU tests and the bench run
on the device for the large configurations) must be the same numbers."""
import numpy as np

from graphnn_amd import synth


def test_splitmix64_known_answers():
    # the first outputs of SplitMix64 seeded with 0 and with 1234567, as published with the generator
    assert [int(x) for x in synth.Stream(0).u64(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    assert [int(x) for x in synth.Stream(1234567).u64(5)] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                                              4593380528125082431, 16408922859458223821]


def test_torch_streams_equal_the_numpy_streams():
    seed = synth.config_seed(5)
    want = synth.Stream(seed)
    want.pos = 12345
    got = synth.torch_u64(seed, 12345, 4097, "cpu").numpy().view(np.uint64)
    assert np.array_equal(got, want.u64(4097))
    u = synth.Stream(seed).uniform(3000)
    assert np.array_equal(synth.torch_uniform(seed, 0, 3000, "cpu").numpy(), u)
    assert np.array_equal(synth.torch_uniform_f32(seed, 3000, "cpu", 0.5, 1.5, chunk=777).numpy(), (0.5 + 1.0 * u).astype(np.float32))
    z = synth.Stream(seed).normal(5000)
    zt = synth.torch_normal_f32(seed, 5000, "cpu", chunk=1024).numpy()
    # same uniforms, float64 routines of another library: equal or the neighbouring float32
    assert np.all(np.abs(zt - z) <= np.spacing(np.abs(z)))
    assert np.mean(zt == z) > 0.99


def test_rmat_on_torch_equals_rmat_on_numpy():
    seed = synth.config_seed(5)
    scale, nnz = 11, 16 << 11
    rp, ci, v = synth.rmat_csr(seed, scale, nnz)
    rp_t, ci_t, v_t = synth.rmat_csr_torch(seed, scale, nnz, "cpu")
    assert np.array_equal(rp, rp_t.numpy()) and np.array_equal(ci, ci_t.numpy()) and np.array_equal(v, v_t.numpy())
    assert rp[-1] == nnz and np.all(np.diff(rp) >= 0)
    # a window of the unsorted edge list, generated on its own
    rows, cols = synth.rmat_edges_torch(seed, scale, nnz, "cpu", lo=1000, hi=3000, chunk=512)
    all_rows, all_cols = synth.rmat_edges_torch(seed, scale, nnz, "cpu")
    assert np.array_equal(rows.numpy(), all_rows.numpy()[1000:3000]) and np.array_equal(cols.numpy(), all_cols.numpy()[1000:3000])
    # the quadrant probabilities (a = 0.57 puts most entries into the low rows and columns)
    top = (all_rows.numpy() < (1 << (scale - 1))).mean()
    assert abs(top - 0.76) < 0.01


def test_erdos_renyi_regular_has_the_same_entries_per_row():
    rp, ci, v = synth.erdos_renyi_csr(synth.config_seed(3), 1000, 10000, regular=True)
    assert np.all(np.diff(rp) == 10) and ci.size == 10000
    for r in range(0, 1000, 97):
        assert np.all(np.diff(ci[rp[r]:rp[r + 1]]) >= 0)
    rp2, ci2, _ = synth.erdos_renyi_csr(synth.config_seed(3), 1000, 10000)
    assert rp2[-1] == 10000 and np.diff(rp2).max() > 10


def test_molecule_sizes_uniform_variant_of_configuration_2():
    b = synth.make_config(2, size_mode="uniform")[0]
    assert b.graph_sizes.min() >= 10 and b.graph_sizes.max() <= 110 and 50 < b.graph_sizes.mean() < 70
    b = synth.make_config(2)[0]
    assert 25 < b.graph_sizes.mean() < 35 and b.graph_sizes.max() <= 110
