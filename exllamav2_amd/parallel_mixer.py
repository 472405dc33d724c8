"""Two mixers side by side on the same layer input: result = left_scale * left(h) + right_scale * right(h).

The halves are ordinary mixers of the stack's registry built with their own tensor prefix (`<layer>.mix.left.*`, `.right.*`), state
key ((layer, "left"), (layer, "right")) and result buffer; the weighted sum is not a launch of its own -- `forward` hands both fp32
results and their scales to the residual step that follows (rmsnorm.SandwichNorm), whose launch reads them."""
from __future__ import annotations


class ParallelMixer:
    def __init__(self, model, key: str, layer_idx: int, left, right, left_scale: float, right_scale: float):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.left, self.right, self.left_scale, self.right_scale = left, right, float(left_scale), float(right_scale)
        self.kv_from = None
        if getattr(left, "kv_from", None) is not None or getattr(right, "kv_from", None) is not None:
            raise ValueError(f"{key}: a half of a parallel mixer keeps its own keys and values")
        if left.out_tag == right.out_tag:
            raise ValueError(f"{key}: the halves need result buffers of their own")

    def load(self, get):
        self.left.load(lambda n, optional=False: get("left." + n, optional))
        self.right.load(lambda n, optional=False: get("right." + n, optional))
        return self

    def weight_bytes(self) -> int:
        return self.left.weight_bytes() + self.right.weight_bytes()

    def make_states(self, pool, dtype) -> dict:
        return {self.left.layer_idx: self.left.make_state(pool, dtype), self.right.layer_idx: self.right.make_state(pool, dtype)}

    def forward(self, xh, rows: int, batch, cache):
        """returns (left result, left scale, right result, right scale): fp32 [rows, width] each"""
        yl = self.left.forward(xh, rows, batch, cache)
        yr = self.right.forward(xh, rows, batch, cache)
        return yl, self.left_scale, yr, self.right_scale
