"""Sizes that the kernels take, as plain numbers: parts check them when a model is put
together (a model that a kernel would refuse at its first step is refused when it is built),
and `ops.py` checks them again before a launch.  Nothing here touches the GPU."""

MAX_HEAD_DIM = 256  # the attention kernels keep a head's elements in four registers per lane
# the widest row whose partial sums (a product taken in slices of K) the residual add + norm adds
# up: 256 threads x 4 elements x NORM_CHUNKS of norm.hip, and a multiple of 4
MAX_SUMMED_NORM_WIDTH = 8192


def check_head_dim(head_dim: int, rotary_dim: int = 0) -> None:
    """Raises ValueError for a head size that the attention kernels refuse."""
    if head_dim <= 0:
        raise ValueError(f"head_dim must be positive, not {head_dim}")
    if head_dim > MAX_HEAD_DIM:
        raise ValueError(f"head_dim {head_dim} is larger than the attention kernels take ({MAX_HEAD_DIM})")
    if rotary_dim and (rotary_dim % 2 or rotary_dim > head_dim):
        raise ValueError(f"a rotation over {rotary_dim} elements does not fit a head_dim of {head_dim} (even, within the head)")
