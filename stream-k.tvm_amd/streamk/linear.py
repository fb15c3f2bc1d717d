"""`torch.nn.Linear`-shaped caller of the Stream-K GEMMs: the step above `streamk_fp16`.

The reference stops at kernel scripts; wrapping them as an operator of a model is its open item
("integrate with BitBLAS", README.md:21).  This module is that wrapper for this library: it owns
the weight in the layout the kernels read ([N, K] fp16 or bfloat16, or packed nibbles + scales), flattens the
leading dimensions of the input into M, and keeps one plan per M it has seen (a decode step calls
with M = batch, a prefill with M = batch * tokens), each taken from the tuned cache when the shape
is in it.  Inference only: the GEMM is not recorded by autograd.
"""
import torch

from . import ops
from .plan import make_plan


class StreamKLinear(torch.nn.Module):
    def __init__(self, in_features, out_features, bias=False, *, weight_format="float16", group=128, zero=8,
                 activation=None, device=None):
        super().__init__()
        if activation not in (None, "relu", "gelu_tanh", "silu"):
            raise ValueError("activation must be None, 'relu', 'gelu_tanh' or 'silu'")
        self.activation = activation  # applied in the GEMM's epilogue, after the bias
        if weight_format not in ("float16", "bfloat16", "q4", "q4_zp"):
            raise ValueError("weight_format must be 'float16', 'bfloat16', 'q4' or 'q4_zp' (one zero point per group)")
        if weight_format in ("q4", "q4_zp") and (group != 128 or in_features % 128):
            raise ValueError("Q4 weights need group == 128 and in_features a multiple of 128")
        if in_features % 8:
            raise ValueError("in_features must be a multiple of 8")
        self.in_features, self.out_features = in_features, out_features
        self.weight_format, self.group, self.zero = weight_format, group, zero
        N, K = out_features, in_features
        # activations, bias and output are bfloat16 with bfloat16 weights, fp16 otherwise
        self.dtype = torch.bfloat16 if weight_format == "bfloat16" else torch.float16
        if weight_format in ("float16", "bfloat16"):
            self.register_buffer("weight", torch.zeros(N, K, dtype=self.dtype, device=device))
        else:
            self.register_buffer("qweight", torch.zeros(N, K // 2, dtype=torch.uint8, device=device))
            self.register_buffer("scales", torch.zeros(N, K // group, dtype=torch.float16, device=device))
            if weight_format == "q4_zp":
                self.register_buffer("zeros", torch.zeros(N, K // group, dtype=torch.float16, device=device))
        self.register_buffer("bias", torch.zeros(N, dtype=self.dtype, device=device) if bias else None)
        self._plans = {}

    @classmethod
    def from_linear(cls, linear, *, weight_format="float16", group=128, zero=8, activation=None):
        """Takes over the weight (and bias) of a torch.nn.Linear; weight_format='q4' / 'q4_zp' quantises
        it with `quantize_q4` (symmetric around `zero` / asymmetric with a zero point per group) on the
        device it lives on."""
        w = linear.weight.detach().to(torch.bfloat16 if weight_format == "bfloat16" else torch.float16).contiguous()
        m = cls(linear.in_features, linear.out_features, linear.bias is not None, weight_format=weight_format,
                group=group, zero=zero, activation=activation, device=w.device)
        if weight_format in ("float16", "bfloat16"):
            m.weight.copy_(w)
        elif weight_format == "q4_zp":
            q, s, z = ops.quantize_q4(w, group=group, asymmetric=True)
            m.qweight.copy_(q)
            m.scales.copy_(s)
            m.zeros.copy_(z)
        else:
            q, s = ops.quantize_q4(w, group=group, zero=zero)
            m.qweight.copy_(q)
            m.scales.copy_(s)
        if linear.bias is not None:
            m.bias.copy_(linear.bias.detach().to(m.dtype))
        return m

    def plan_for(self, M):
        """The plan a call with M rows runs (what forward's operator call resolves to)."""
        p = self._plans.get(M)
        if p is None:
            dtype = self.weight_format
            p = self._plans[M] = make_plan(M, self.out_features, self.in_features, dtype, "nt")
        return p

    @torch.no_grad()
    def forward(self, x):
        """Calls the registered operators (torch.ops.streamk.gemm_*) with tensors and plain values only, so the
        module traces under torch.compile without a graph break; the operator keeps one plan per M it has seen
        (from the tuned cache where the shape is in it)."""
        if x.dtype != self.dtype or x.shape[-1] != self.in_features:
            raise ValueError(f"input must be {self.dtype} [..., {self.in_features}], got {x.dtype} {tuple(x.shape)}")
        lead = x.shape[:-1]
        a = x.reshape(-1, self.in_features)
        if a.shape[0] == 0:
            return x.new_zeros(*lead, self.out_features)
        # bias and activation are applied in the GEMM's epilogue (fp32, before the rounding to C's type)
        act = self.activation or "none"
        if self.weight_format == "float16":
            c = torch.ops.streamk.gemm_f16(a, self.weight, "nt", "", self.bias, act)
        elif self.weight_format == "bfloat16":
            c = torch.ops.streamk.gemm_bf16(a, self.weight, "nt", "", self.bias, act)
        else:
            zeros = self.zeros if self.weight_format == "q4_zp" else None
            c = torch.ops.streamk.gemm_q4(a, self.qweight, self.scales, zeros, self.zero, self.group, False, "",
                                          self.bias, act)
        return c.view(*lead, self.out_features)

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"weight_format={self.weight_format}, activation={self.activation}")
