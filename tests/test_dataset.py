"""Host-side data formats either side of the operators: APR state pickling and files (BindAPR.hpp:67-131,
io_api.py), data sets and collate functions (apr_models/utils/dataset.py).  CPU only; the StarDist targets of
StarDistDataset need the device kernels and are covered by the GPU test at the end."""
import os
import pickle

import numpy as np
import pytest
import torch

import pyapr
from apr_models.utils import (APRDataset, StarDistDataset, collate_intensity, collate_intensity_and_labels,
                              collate_stardist, split_dataset)


def _apr(seed, shape=(12, 20, 24)):
    rng = np.random.default_rng(seed)
    img = (rng.random(shape) * 4000).astype(np.uint16)
    img[: shape[0] // 2] //= 8
    return pyapr.converter.get_apr(img)


def _same_structure(a, b):
    for ia, ib in ((a.iterator(), b.iterator()), (a.tree_iterator(), b.tree_iterator())):
        assert np.array_equal(ia.xz_end_vec, ib.xz_end_vec) and np.array_equal(ia.y_vec, ib.y_vec)
        assert np.array_equal(ia.level_xz_vec, ib.level_xz_vec)
    assert a.shape() == b.shape() and a.level_max() == b.level_max() and a.level_min() == b.level_min()


def test_pickle_state_is_the_reference_tuple():
    apr, _ = _apr(0)
    apr.name = "sample"
    state = apr.__getstate__()
    # BindAPR.hpp:72-80: org_dims(0..2) = (y, x, z), parameters, xz_end_vec u64, y_vec u16, tree xz_end_vec, tree y_vec
    assert state[:3] == (24, 20, 12)
    assert state[4].dtype == np.uint64 and state[5].dtype == np.uint16
    assert state[6].dtype == np.uint64 and state[7].dtype == np.uint16
    assert state[5].shape[0] == apr.total_number_particles() and state[7].shape[0] == apr.total_number_tree_particles()
    back = pickle.loads(pickle.dumps(apr))
    _same_structure(apr, back)
    assert back.name == "sample" and back.get_parameters().rel_error == apr.get_parameters().rel_error
    with pytest.raises(RuntimeError):
        pyapr.APR().__getstate__()                      # "APR not initialized", BindAPR.hpp:68-70
    with pytest.raises(RuntimeError):
        pyapr.APR().__setstate__((1, 2, 3))             # invalid state size, BindAPR.hpp:93-94


def test_particle_levels_follow_the_level_ranges():
    apr, _ = _apr(1)
    lev = apr.particle_levels()
    it = apr.iterator()
    assert lev.shape[0] == apr.total_number_particles()
    for level in range(it.level_min(), it.level_max() + 1):
        for z in range(it.z_num(level)):
            for x in range(0, it.x_num(level), 3):
                b = it.begin(level, z, x)
                assert np.all(lev[b:it.end()] == level)


def test_file_round_trip(tmp_path):
    apr, parts = _apr(2)
    f = str(tmp_path / "a.apr")
    pyapr.io.write(f, apr, parts)
    assert os.path.isfile(f)                                            # the name is used as given
    labels = (parts > parts.mean()).astype(np.uint16)
    pyapr.io.write_particles(f, labels, parts_name="labels")
    pyapr.io.write_particles(f, np.ones(apr.total_number_tree_particles(), np.float32), parts_name="mean", tree=True)
    back, p = pyapr.io.read(f)
    _same_structure(apr, back)
    assert p.dtype == np.float32 and np.array_equal(p, parts)
    assert np.array_equal(pyapr.io.read_particles(f, parts_name="labels"), labels)
    assert pyapr.io.get_particle_names(f) == ["particles", "labels"]
    assert pyapr.io.get_particle_names(f, tree=True) == ["mean"]
    assert pyapr.io.get_particle_type(f, parts_name="labels") == "uint16"
    _same_structure(apr, pyapr.io.read_apr(f))
    with pytest.raises(ValueError):
        pyapr.io.read(str(tmp_path / "missing.apr"))                    # io_api.py:55-56
    with pytest.raises(ValueError):
        pyapr.io.read(f, parts_name="nope")
    with pytest.raises(ValueError):
        pyapr.io.write(f, apr, parts[:-1])
    with pytest.raises(ValueError):
        pyapr.io.read(f, parts=np.zeros(0, np.uint16))                  # type must match the file


def _write_set(tmp_path, n):
    out = []
    for i in range(n):
        apr, parts = _apr(10 + i, shape=(8 + 2 * i, 16, 20 + 4 * i))
        labels = (np.arange(parts.shape[0]) % 3).astype(np.uint16)
        f = str(tmp_path / f"s{i}.apr")
        pyapr.io.write(f, apr, parts)
        pyapr.io.write_particles(f, labels, parts_name="labels")
        out.append((apr, parts, labels))
    return out


def test_apr_dataset_and_collates(tmp_path):
    samples = _write_set(tmp_path, 3)
    ds = APRDataset(str(tmp_path), labels_name="labels")
    assert len(ds) == 3
    items = [ds[i] for i in range(3)]
    for (apr, parts, labs), (a0, p0, l0) in zip(items, samples):
        _same_structure(apr, a0)
        assert np.array_equal(parts, p0) and np.array_equal(labs, l0)
    lens = [s[1].shape[0] for s in samples]
    assert len(set(lens)) == 3                                          # a ragged batch
    n_max = max(lens)

    aprs, x, y = collate_intensity_and_labels()(items)
    assert x.shape == (3, 1, n_max) and x.dtype == torch.float32 and y.shape == (3, 1, n_max) and y.dtype == torch.float32
    for i, (_, p0, l0) in enumerate(samples):
        assert torch.equal(x[i, 0, :lens[i]], torch.from_numpy(p0)) and not x[i, 0, lens[i]:].any()
        assert torch.equal(y[i, 0, :lens[i]], torch.from_numpy(l0.astype(np.float32))) and not y[i, 0, lens[i]:].any()

    aprs, x, y = collate_intensity_and_labels(labels_drop_channel_dim=True, label_dtype=torch.long, input_levels=True)(items)
    assert x.shape == (3, 2, n_max) and y.shape == (3, n_max) and y.dtype == torch.long
    for i, (a0, _, l0) in enumerate(samples):
        want = a0.particle_levels().astype(np.float32) * np.float32(1 / a0.level_max())
        assert torch.equal(x[i, 1, :lens[i]], torch.from_numpy(want)) and not x[i, 1, lens[i]:].any()
        assert torch.equal(y[i, :lens[i]], torch.from_numpy(l0.astype(np.int64)))

    aprs, x = collate_intensity()(items)
    assert len(aprs) == 3 and x.shape == (3, 1, n_max) and torch.equal(x[1, 0, :lens[1]], torch.from_numpy(samples[1][1]))

    unlabelled = APRDataset([str(tmp_path)], transform=lambda p, l=None: (p * 2, l))
    apr, parts, labs = unlabelled[0]
    assert labs is None and np.array_equal(parts, samples[0][1] * 2)


def test_split_dataset(tmp_path):
    _write_set(tmp_path, 3)
    ds = APRDataset(str(tmp_path), labels_name="labels")
    np.random.seed(0)
    a, b = split_dataset(ds, 1, transforms=[None, lambda p, l=None: (p + 1, l)])
    assert len(a) == 1 and len(b) == 2 and sorted(a.indices + b.indices) == [0, 1, 2]
    _, parts, _ = b[0]
    assert np.array_equal(parts, ds[b.indices[0]][1] + 1)
    with pytest.raises(AssertionError):
        split_dataset(ds, [1, 1], transforms=[None, None])


def test_collate_stardist_pads_every_sample_from_its_own_length():
    rng = np.random.default_rng(5)
    data = []
    for n in (7, 4, 9):
        data.append((object.__new__(pyapr.APR), rng.random(n).astype(np.float32), rng.random((n, 6)).astype(np.float32),
                     rng.random(n).astype(np.float32)))
    aprs, x, prob, dist = collate_stardist()(data)
    assert x.shape == (3, 1, 9) and prob.shape == (3, 1, 9) and dist.shape == (3, 6, 9)
    for i, (_, p, d, pr) in enumerate(data):
        n = p.shape[0]
        assert torch.equal(x[i, 0, :n], torch.from_numpy(p)) and torch.equal(prob[i, 0, :n], torch.from_numpy(pr))
        assert torch.equal(dist[i, :, :n], torch.from_numpy(d).T)
        assert not x[i, 0, n:].any() and not prob[i, 0, n:].any() and not dist[i, :, n:].any()
    aprs, x, prob, dist = collate_stardist()([(a, p, None, None) for a, p, _, _ in data])
    assert prob is None and dist is None and x.shape == (3, 1, 9)


def test_stardist_dataset_without_labels(tmp_path, capsys):
    _write_set(tmp_path, 2)
    ds = StarDistDataset(rays=None, data_dir=str(tmp_path), label_dir=str(tmp_path / "none"))
    assert "does not exist" in capsys.readouterr().out
    apr, parts, dist, prob = ds[0]
    assert dist is None and prob is None and parts.shape[0] == apr.total_number_particles()


def test_stardist_dataset_with_labels_refuses_loader_workers(tmp_path, monkeypatch):
    """The label targets are computed on the GPU, which a DataLoader worker process cannot use: a clear error
    instead of 'Cannot re-initialize CUDA in forked subprocess' (the reference's CPU loops work in workers)."""
    (tmp_path / "img").mkdir(); (tmp_path / "lab").mkdir()
    img = (np.random.default_rng(0).random((6, 12, 12)) * 1000).astype(np.uint16)
    np.save(tmp_path / "img" / "v0.npy", img)
    np.save(tmp_path / "lab" / "v0_seg.npy", np.zeros(img.shape, np.uint16))
    rays = np.array([[1, 0, 0]], np.float32)
    ds = StarDistDataset(rays, str(tmp_path / "img"), str(tmp_path / "lab"), label_tag="_seg", pixels=True, file_ext="*.npy")
    monkeypatch.setattr(torch.utils.data, "get_worker_info", lambda: object())
    with pytest.raises(RuntimeError, match="num_workers=0"):
        ds[0]


@pytest.mark.gpu
def test_stardist_dataset_targets_from_images(tmp_path):
    """pixels=True: image -> APR on the fly, targets from the device kernels; checked against the oracle."""
    from oracle import oracle
    rng = np.random.default_rng(3)
    (tmp_path / "img").mkdir(); (tmp_path / "lab").mkdir()
    for i in range(2):
        img = (rng.random((10, 24, 28)) * 3000).astype(np.uint16)
        lab = np.zeros(img.shape, np.uint16)
        lab[2:8, 4:15, 5:20] = 1
        lab[3:9, 16:22, 8:26] = 2
        np.save(tmp_path / "img" / f"v{i}.npy", img)
        np.save(tmp_path / "lab" / f"v{i}_seg.npy", lab)
    rays = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [0, -1, 0], [0.5, 0.5, -0.7]], np.float32)
    ds = StarDistDataset(rays, str(tmp_path / "img"), str(tmp_path / "lab"), label_tag="_seg", pixels=True, file_ext="*.npy",
                         prob_fn=lambda lab: (lab > 0).astype(np.float32))
    items = [ds[0], ds[1]]
    for i, (apr, parts, dist, prob) in enumerate(items):
        lab = np.load(tmp_path / "lab" / f"v{i}_seg.npy")
        r = torch.from_numpy(rays)
        want = oracle.labels_to_dist(apr, torch.from_numpy(lab), r[:, 0], r[:, 1], r[:, 2], 0)
        assert np.array_equal(dist, want.numpy())
        assert np.array_equal(prob, oracle.sample_image_max(apr, torch.from_numpy(lab > 0).float(), 0).numpy())
    aprs, x, prob, dist = collate_stardist()(items)
    n_max = max(a.total_number_particles() for a in aprs)
    assert x.shape == (2, 1, n_max) and prob.shape == (2, 1, n_max) and dist.shape == (2, 5, n_max)
