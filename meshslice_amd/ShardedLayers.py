"""``ShardedFFLayer``: a linear layer whose forward, backward-data and backward-weight passes are the
three dataflows of the 2-D GEMM (reference ShardedLayers.py:20-83).

The reference wires the passes with ``jax.custom_vjp``; here a ``torch.autograd.Function`` plays that
role, so ``layer.forward(x)`` is differentiable with respect to ``x`` and ``layer.weight``:

    'os' : y = OS(x, w)   dx = LS(dy, w)   dw = RS(x, dy)        w stored [in, out]
    'ls' : y = LS(x, w)   dx = OS(dy, w)   dw = RS(dy, x)        w stored [out, in]
    'rs' : y = RS(x, w)   dx = LS(w, dy)   dw = OS(x, dy)        w stored [in, out], x stored [in, tokens]

The layer norm, attention and transformer-block classes of the reference file are not part of this
build (they contain no sliced GEMM).
"""
from __future__ import annotations

from functools import partial

import torch

from .TensorParallel import SPMD, createMultihostMatrix
from .mesh import Mesh, NamedSharding, PartitionSpec as P


class ShardedFFLayer:
    def __init__(self, mesh: Mesh, algorithm: str, dataflow: str, ksplit: int, in_dim: int, out_dim: int,
                 blocksize: int = 8, seed: int = 0, device="cuda"):
        if dataflow not in ("os", "ls", "rs"):
            raise ValueError(f"dataflow must be 'os', 'ls' or 'rs', got {dataflow!r}")
        self.mesh = mesh
        row, col = mesh.axis_names
        self.algorithm = algorithm
        self.dataflow = dataflow
        self.ksplit = ksplit
        self.blocksize = blocksize
        shape = [out_dim, in_dim] if dataflow == "ls" else [in_dim, out_dim]   # reference :33-36
        self.weight = createMultihostMatrix(mesh, NamedSharding(mesh, P(row, col)), shape, seed=seed, device=device)
        builder = SPMD(mesh, algorithm, blocksize)
        OS, LS, RS = builder.OS(ksplit), builder.LS(ksplit), builder.RS(ksplit)
        # (forward, dx(dy, x, w), dw(dy, x, w)) per dataflow, reference :41-81
        table = {
            "os": (OS, lambda dy, x, w: LS(dy, w), lambda dy, x, w: RS(x, dy)),
            "ls": (LS, lambda dy, x, w: OS(dy, w), lambda dy, x, w: RS(dy, x)),
            "rs": (RS, lambda dy, x, w: LS(w, dy), lambda dy, x, w: OS(x, dy)),
        }
        fwd, bwd_x, bwd_w = table[dataflow]

        class _Compute(torch.autograd.Function):
            @staticmethod
            def forward(ctx, x, w):
                ctx.save_for_backward(x, w)
                return fwd(x, w)

            @staticmethod
            def backward(ctx, dy):
                x, w = ctx.saved_tensors
                dy = dy.contiguous()
                dx = bwd_x(dy, x, w) if ctx.needs_input_grad[0] else None
                dw = bwd_w(dy, x, w) if ctx.needs_input_grad[1] else None
                return dx, dw

        self.compute = _Compute.apply
        self.forward = partial(self._forward)

    def _forward(self, x, w=None):
        return self.compute(x, self.weight if w is None else w)
