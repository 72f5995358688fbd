"""Loader of the fixtures under tests/golden (numpy.load without pickle)."""

from pathlib import Path

import numpy as np
import torch

GOLDEN = Path(__file__).resolve().parent / "golden"


def load(name):
    data = np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
    result = {}
    for key in data.files:
        array = data[key]
        if array.dtype == np.uint16:   # bf16 bit patterns
            result[key] = torch.from_numpy(array.astype(np.int16)).view(torch.bfloat16)
        elif array.ndim == 0:
            result[key] = float(array)
        else:
            result[key] = torch.from_numpy(array)
    return result
