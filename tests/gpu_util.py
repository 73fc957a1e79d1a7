"""Helpers for the GPU parity tests: load the package, move numpy arrays to the device."""
import importlib
import sys

import numpy as np


def espdl():
    return importlib.import_module("esp-dl_amd")


def announce(msg):
    """Name the case before each GPU step so a fault can be attributed."""
    print("[gpu-case] " + msg, flush=True)
    sys.stdout.flush()


def to_dev(a):
    import torch
    if a is None:
        return None
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_host(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()
