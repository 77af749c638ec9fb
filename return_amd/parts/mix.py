"""What becomes of the residual stream after a layer when it is not simply the layer's result.

"depth_weighted": with X_0 the embedding's output and X_j the result of the j-th layer run, the stream that goes
on after the n-th run is  sum_{j <= n} w[j] X_j  with one stored weight per term (n + 1 of them). The sum is
formed in 32-bit, terms in order; the next layer's first norm may be formed in the same kernel.
"""
from __future__ import annotations

import torch

from .registry import register_part


class DepthWeightedStream:
    @staticmethod
    def tensor_shapes(params):
        return {"weights": (params["count"],)}

    @staticmethod
    def random_init(params, role):
        n = int(params["count"])

        def draw(shape, gen):
            # most of the weight on the newest result, the rest spread over the older ones
            w = 0.3 * torch.rand(*shape, generator=gen, dtype=torch.float32, device=gen.device) / max(n - 1, 1)
            w[-1] = 0.8 + 0.2 * torch.rand(1, generator=gen, dtype=torch.float32, device=gen.device)
            return w
        return draw

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.count = int(params["count"])
        self.weights = rt.vector32(tensors["weights"])

    takes_normed = True         # forward(..., post=Normed): the newest result still lacks that output

    def forward(self, results, count, out, norm=None, post=None):
        """post: a Normed that is still to be added into the newest result, results[count - 1] (a kernel set with
        post_norm_mix does that in the same pass over the rows)."""
        ops = self.rt.ops
        if count != self.count:
            raise ValueError(f"a weighted sum over {self.count} results was handed {count}")
        fused = post is not None and hasattr(ops, "post_norm_mix")
        if post is not None and not fused:
            ops.post_norm_add(results[count - 1], post.tensor, post.weight, post.eps)
        if norm is not None and hasattr(norm, "weight") and hasattr(norm, "eps"):
            x = self.rt.empty(out.shape[0], out.shape[1])
            if fused:
                ops.post_norm_mix(results, count, self.weights, post.tensor, post.weight, post.eps, out, norm.weight, norm.eps, x)
            else:
                ops.depth_mix(results, count, self.weights, out, norm.weight, norm.eps, x)
            return x
        if fused:
            ops.post_norm_mix(results, count, self.weights, post.tensor, post.weight, post.eps, out)
        else:
            ops.depth_mix(results, count, self.weights, out)
        return None


register_part("stream_mix", "depth_weighted", DepthWeightedStream)
