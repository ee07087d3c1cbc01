"""Data sets and batch collation for the particle-space models (apr_models/apr_models/utils/__init__.py)."""
from . import dataset
from .dataset import (APRDataset, StarDistDataset, SplitDataset, split_dataset, collate_intensity,
                      collate_intensity_and_labels, collate_stardist)

__all__ = ["dataset", "APRDataset", "StarDistDataset", "SplitDataset", "split_dataset", "collate_intensity",
           "collate_intensity_and_labels", "collate_stardist"]
