"""Data sets of APR files and the collate functions that turn ragged samples into the padded
``[batch, channels, max particles]`` tensors the operators take (apr_models/apr_models/utils/dataset.py:12-192).

Same class names, constructor arguments and return tuples as the reference.  Differences, all at the file layer:
APR files are the ``.npz`` containers of :mod:`pyapr.io` (LibAPR's HDF5 reader is not part of the reference tree);
images are read from ``.npy`` or, through Pillow, multi-page TIFF (the reference uses scikit-image); the StarDist
targets come from the device kernels of :mod:`pyapr.aprnet.stardist_utils`.
"""
from glob import glob
from os.path import basename, exists, join, splitext

import numpy as np
import torch
from torch.utils.data import Dataset, Subset

import pyapr
from pyapr.aprnet import stardist_utils


def _glob_dirs(dirs, pattern):
    if isinstance(dirs, str):
        return sorted(glob(join(dirs, pattern)))
    return [f for d in dirs for f in sorted(glob(join(d, pattern)))]


def imread(path):
    """Image file -> numpy array; a multi-page TIFF becomes (pages, rows, columns)."""
    if path.endswith(".npy"):
        return np.load(path, allow_pickle=False)
    from PIL import Image, ImageSequence
    with Image.open(path) as im:
        pages = [np.array(page) for page in ImageSequence.Iterator(im)]
    return pages[0] if len(pages) == 1 else np.stack(pages)


class APRDataset(Dataset):
    """``(apr, parts, labels or None)`` per file (dataset.py:12-38)."""

    def __init__(self, root_dir, parts_name="particles", labels_name=None, transform=None):
        self.root_dir = root_dir
        self.file_list = _glob_dirs(root_dir, "*.apr")
        self.parts_name = parts_name
        self.labels_name = labels_name
        self.transform = transform

    def __len__(self):
        return len(self.file_list)

    def __getitem__(self, index):
        path = self.file_list[index]
        apr, parts = pyapr.io.read(path, parts_name=self.parts_name)
        if self.labels_name:
            labs = pyapr.io.read_particles(path, parts_name=self.labels_name)
            if self.transform:
                parts, labs = self.transform(parts, labs)
            return apr, parts, labs
        if self.transform:
            parts, _ = self.transform(parts)
        return apr, parts, None


class SplitDataset(Dataset):
    """View of a data set with its own transform, applied after the transform of the wrapped set (the wrapper
    that split_dataset builds its subsets from, dataset.py:134; the reference never defines the class it names there)."""

    def __init__(self, dataset, transform=None):
        self.dataset = dataset
        self.transform = transform

    def __len__(self):
        return len(self.dataset)

    def __getitem__(self, index):
        apr, parts, labs = self.dataset[index]
        if self.transform:
            if labs is not None:
                parts, labs = self.transform(parts, labs)
            else:
                parts, _ = self.transform(parts)
        return apr, parts, labs


class StarDistDataset(Dataset):
    """``(apr, parts, dist, prob)`` per file; ``dist`` [particles, rays] and ``prob`` [particles] are None without a
    label directory (dataset.py:41-104).  With ``pixels=True`` the files are images, optionally cropped at random to
    ``crop_size``, converted to an APR on the fly with ``rel_error`` fixed or drawn uniformly from a (low, high) pair."""

    def __init__(self, rays, data_dir, label_dir=None, label_tag="", parts_name="particles", pixels=False, file_ext=None,
                 crop_size=None, rel_error=0.1, transform=None, prob_fn=None):
        self.data_dir = data_dir
        self.label_dir = label_dir
        self.pixels = pixels
        self.rel_error = rel_error
        self.crop_size = crop_size
        file_ext = file_ext or ("*.tif" if pixels else "*.apr")
        self.file_list = _glob_dirs(data_dir, file_ext)
        self.labels = label_dir is not None and exists(label_dir)
        if not self.labels:
            print(f"labels directory {label_dir} does not exist - StarDistDataset will not yield ground truth data")
        self.rays = rays
        self.parts_name = parts_name
        self.label_tag = label_tag
        self.transform = transform
        self.prob_fn = prob_fn          # forwarded to get_prob_apr; None = stardist's edt_prob as in the reference

    def __len__(self):
        return len(self.file_list)

    def _label_path(self, data_path):
        stem = splitext(basename(data_path))[0]
        for ext in (".tif", ".npy"):
            p = join(self.label_dir, f"{stem}{self.label_tag}{ext}")
            if exists(p):
                return p
        raise FileNotFoundError(f"no label image for {data_path} in {self.label_dir}")

    def __getitem__(self, index):
        data_path = self.file_list[index]
        window = None
        if self.pixels:
            img = imread(data_path)
            par = pyapr.APRParameters()
            par.rel_error = self.rel_error if isinstance(self.rel_error, float) else float(np.random.uniform(*self.rel_error))
            par.auto_parameters = True
            if self.crop_size is not None:
                assert len(self.crop_size) == 3
                sz = [min(self.crop_size[i], img.shape[i]) for i in range(3)]
                corner = np.random.randint(0, [max(img.shape[i] - sz[i], 1) for i in range(3)])
                window = tuple(slice(int(corner[i]), int(corner[i]) + sz[i]) for i in range(3))
                img = np.ascontiguousarray(img[window])
            apr, parts = pyapr.converter.get_apr(img, params=par, verbose=False)
        else:
            apr, parts = pyapr.io.read(data_path, parts_name=self.parts_name)

        dist = prob = None
        if self.labels:
            # The label targets are computed on the GPU (the reference has CPU loops, utils.hpp:86-333): a DataLoader
            # worker process has no usable GPU context (CUDA cannot be re-initialised after fork, and every spawned
            # worker would open a context of its own), so this data set is for num_workers = 0.
            if torch.utils.data.get_worker_info() is not None:
                raise RuntimeError("StarDistDataset computes its label targets on the GPU: use DataLoader(num_workers=0)")
            label_image = imread(self._label_path(data_path))
            if window is not None:
                label_image = np.ascontiguousarray(label_image[window])
            dist = stardist_utils.labels_to_dist(apr, label_image, self.rays)
            prob = stardist_utils.get_prob_apr(apr, label_image, prob_fn=self.prob_fn)
        if self.transform:
            parts = self.transform(parts)
        return apr, parts, dist, prob


def split_dataset(dataset, sizes, transforms=None):
    """Random disjoint subsets of sizes ``[*sizes, len(dataset) - sum(sizes)]``, each with its own transform
    (dataset.py:107-135)."""
    if isinstance(sizes, int):
        sizes = [sizes]
    n_subsets = len(sizes) + 1
    if isinstance(transforms, list):
        assert len(transforms) == n_subsets, \
            "Number of provided transforms (%d) does not match number of subsets (%d)" % (len(transforms), n_subsets)
    else:
        transforms = [transforms] * n_subsets
    indices = list(range(len(dataset)))
    np.random.shuffle(indices)
    cuts = [0] + [int(c) for c in np.cumsum(sizes)] + [len(dataset)]
    return tuple(Subset(SplitDataset(dataset, transform=transforms[i]), indices[cuts[i]:cuts[i + 1]])
                 for i in range(n_subsets))


def _pad_rows(rows, channels, dtype):
    """rows: one [len_i] or [channels, len_i] array per sample -> zero-padded [batch, channels, max len]."""
    out = torch.zeros((len(rows), channels, max(r.shape[-1] for r in rows)), dtype=dtype)
    for i, r in enumerate(rows):
        out[i, :, :r.shape[-1]] = torch.as_tensor(np.asarray(r)).to(dtype)
    return out


class collate_intensity_and_labels:
    """-> (aprs, intensities [B, 1 or 2, Nmax] float32, labels [B, 1, Nmax] or [B, Nmax]); with ``input_levels`` the
    second channel is particle level / level_max (dataset.py:138-160).  Labels pass through float32 before the cast to
    ``label_dtype``, as in the reference."""

    def __init__(self, labels_drop_channel_dim=False, label_dtype=torch.float32, input_levels=False):
        self.labels_drop_channel_dim = labels_drop_channel_dim
        self.label_dtype = label_dtype
        self.input_levels = input_levels

    def __call__(self, data):
        aprs, parts, labs = (list(v) for v in zip(*data))
        n_max = max(a.total_number_particles() for a in aprs)
        intensities = torch.zeros((len(aprs), 2 if self.input_levels else 1, n_max), dtype=torch.float)
        labels = torch.zeros((len(aprs), 1, n_max), dtype=self.label_dtype)
        for i, (a, p, l) in enumerate(zip(aprs, parts, labs)):
            intensities[i, 0, :len(p)] = torch.from_numpy(np.asarray(p, dtype=np.float32))
            if self.input_levels:
                lev = a.particle_levels().astype(np.float32) * np.float32(1 / a.level_max())
                intensities[i, 1, :len(lev)] = torch.from_numpy(lev)
            labels[i, 0, :len(l)] = torch.from_numpy(np.asarray(l).astype(np.float32)).to(self.label_dtype)
        return aprs, intensities, labels[:, 0] if self.labels_drop_channel_dim else labels


class collate_intensity:
    """-> (aprs, intensities [B, 1, Nmax] float32) (dataset.py:163-171)."""

    def __call__(self, data):
        aprs, parts = [list(v) for v in zip(*data)][:2]
        return aprs, _pad_rows([np.asarray(p, dtype=np.float32) for p in parts], 1, torch.float)


class collate_stardist:
    """-> (aprs, intensities [B, 1, Nmax], prob [B, 1, Nmax], dist [B, rays, Nmax]) or ``(..., None, None)`` without
    targets (dataset.py:174-192).  Every sample is padded from its own length; the reference slices all targets with
    the length of the last sample of the batch (:187-188) and therefore only accepts batches of equal lengths, where
    the two agree."""

    def __call__(self, data):
        aprs, parts, dist, prob = (list(v) for v in zip(*data))
        intensities = _pad_rows([np.asarray(p, dtype=np.float32) for p in parts], 1, torch.float)
        if dist[0] is None:
            return aprs, intensities, None, None
        n_max = intensities.shape[-1]
        prob_t = torch.zeros((len(aprs), 1, n_max), dtype=torch.float)
        dist_t = torch.zeros((len(aprs), dist[0].shape[1], n_max), dtype=torch.float)
        for i, (d, p) in enumerate(zip(dist, prob)):
            prob_t[i, 0, :len(p)] = torch.as_tensor(p, dtype=torch.float)
            dist_t[i, :, :len(p)] = torch.as_tensor(d, dtype=torch.float).transpose(1, 0)
        return aprs, intensities, prob_t, dist_t
