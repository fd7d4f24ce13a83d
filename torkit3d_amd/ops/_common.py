"""Small helpers shared by the op wrappers."""
import torch

CUDA_ONLY = "Only support cuda currently."


def with_batch_dim(cloud):
    """[N, 3] -> [1, N, 3]; batched clouds pass through."""
    return cloud[None] if cloud.dim() == 2 else cloud


def rows_of_points(cloud, channels_first):
    """View of the cloud as [B, N, 3] (a transposed view when it arrives as [B, 3, N])."""
    return cloud.transpose(1, 2) if channels_first else cloud


def on_gpu(*tensors):
    """Contiguous versions of the tensors, which must live on a GPU (the reference's
    wrappers assert this with the same message)."""
    for t in tensors:
        assert t.is_cuda, CUDA_ONLY
    return tuple(t.contiguous() for t in tensors)


class NoGradient(torch.autograd.Function):
    """Base of the index-producing ops: every output is marked non-differentiable and
    backward hands ``None`` to every input."""

    @staticmethod
    def run(*args):
        raise NotImplementedError

    @classmethod
    def forward(cls, ctx, *args):
        ctx.arity = len(args)
        out = cls.run(*args)
        ctx.mark_non_differentiable(*(out if isinstance(out, (tuple, list)) else (out,)))
        return tuple(out) if isinstance(out, list) else out

    @staticmethod
    def backward(ctx, *grad_outputs):
        return (None,) * ctx.arity
