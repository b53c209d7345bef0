"""Dense feed-forward with one up projection: down(act(up h)), no gate and no biases.
``activation``: "relu2" (the square of relu), "gelu_tanh" or "silu"; computed in float32 inside the kernel.  For few rows
the activation is the epilogue of the up projection (applied to the product as rounded to its dtype, so the result is the
same bits as the product followed by the activation kernel)."""
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import FeedForward, register_part
from .linear import linear, own_kernel_applies


@register_part("feed_forward", "dense_act")
class DenseActFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 up_name: str = "up", down_name: str = "down"):
        super().__init__(name, runtime)
        if activation not in ops.ACTIVATIONS:
            raise ValueError("dense feed-forward: activation %r (have %s)" % (activation, ", ".join(sorted(ops.ACTIVATIONS))))
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.activation = activation
        self.up_name, self.down_name = name + up_name, name + down_name
        self.w_up = self.w_down = None

    def weight_specs(self):
        return {self.up_name: WeightSpec((self.intermediate_size, self.hidden_size)),
                self.down_name: WeightSpec((self.hidden_size, self.intermediate_size))}

    def load_weights(self, tensors):
        self.w_up, self.w_down = tensors[self.up_name], tensors[self.down_name]

    def forward(self, h, ctx):
        rt = self.runtime
        T = h.shape[0]
        u = ctx.ws.buffer("ffn_up", (T, self.intermediate_size), rt.dtype)
        if h.dtype == self.w_up.dtype and own_kernel_applies(T, h.dtype, self.w_up.dtype, u.dtype, rt.gemm_impl):
            ops.gemm_nt(h, self.w_up, u, activation=self.activation)      # few rows: the activation is the product's epilogue
        else:
            linear(h, self.w_up, u, rt.gemm_impl, ws=ctx.ws)
            ops.activation(u, u, self.activation)
        y = ctx.ws.buffer("ffn_out", (T, self.hidden_size), rt.dtype)
        linear(u, self.w_down, y, rt.gemm_impl, ws=ctx.ws)
        return y
