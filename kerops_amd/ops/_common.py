"""Helpers shared by the op wrappers."""
import torch


def next_power_of_2(n):
    """Smallest power of two >= n (n >= 1)."""
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


def numel_no_channels(x):
    return x.numel() // x.shape[1]


def require_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                'kerops_amd ops run only on a ROCm device (got a tensor on '
                f'{t.device}); there is no CPU path'
            )


def cl3d(t):
    return t.is_contiguous(memory_format=torch.channels_last_3d)
