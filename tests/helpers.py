"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

DEV = "cuda:0"


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def to_np(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def torch_dtype(np_dtype):
    return {np.dtype(np.float16): torch.float16, np.dtype(np.float32): torch.float32}[np.dtype(np_dtype)]


from oracle.model_io import oracle_weights_from_message  # noqa: E402,F401
