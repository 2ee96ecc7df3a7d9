"""Loads the committed fixtures of tests/golden/ (plain numpy arrays, no pickles)."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def bf16(a):
    """uint16 bit patterns -> bf16 tensor."""
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a))
