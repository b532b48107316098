"""The three masks the causal linear-attention path looks at (own counterpart of the parts
of ``fast_transformers/masking.py:97-206`` that ``CausalLinearAttention`` and the encoder
use: the ``lower_triangular`` flag, ``float_matrix`` of a length mask, default masks)."""
import torch


class FullMask:
    """Every query may look at every key (``masking.py:117-168``): not causal."""
    lower_triangular = False

    def __init__(self, N, M=None, device="cpu"):
        self.shape = (N, M or N)
        self.device = device

    @property
    def bool_matrix(self):
        return torch.ones(self.shape, dtype=torch.bool, device=self.device)


class TriangularCausalMask:
    """Query i sees keys j <= i (``masking.py:195-206``)."""
    lower_triangular = True

    def __init__(self, N, device="cpu"):
        self.shape = (N, N)
        self.device = device

    @property
    def bool_matrix(self):
        return torch.tril(torch.ones(self.shape, dtype=torch.bool, device=self.device))


class LengthMask:
    """Per-sequence valid lengths (``masking.py:171-192``): ``float_matrix[n, s]`` is 1 for
    s < lengths[n]."""
    lower_triangular = False

    def __init__(self, lengths, max_len=None, device=None):
        self.lengths = lengths.clone() if device is None else lengths.to(device)
        self.max_len = int(max_len if max_len is not None else self.lengths.max())

    @property
    def bool_matrix(self):
        idx = torch.arange(self.max_len, device=self.lengths.device)
        return idx[None, :] < self.lengths[:, None]

    @property
    def float_matrix(self):
        return self.bool_matrix.float()
