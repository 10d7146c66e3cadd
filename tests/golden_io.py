"""Loader for the fixtures under tests/golden/ (plain numpy arrays, no pickles)."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def bf16(arr):
    return torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)


def t(arr):
    return torch.from_numpy(np.ascontiguousarray(arr))
