"""RMSNorm operator — mirror of archive/ktransformers/operators/layernorm.py:47-87 (class RMSNorm): `forward(x)` is
forward_native's math, `forward(x, batch_size_tensor)` flashinfer's rmsnorm, `forward(x, batch_size_tensor, residual)` the
in-place fused add + norm returning (x, residual).  All three run csrc/ktx_ops.hip."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class RMSNorm(BaseInjectedModule):
    def __init__(self, key, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda",
                 generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)

    def load(self):
        w = self.gguf_loader.load_tensor(self.key + ".weight", device=self.device)
        self.orig_module.weight = nn.Parameter(w.to(torch.bfloat16), requires_grad=False)

    def forward(self, x: torch.Tensor, batch_size_tensor: torch.Tensor = None, residual: torch.Tensor = None):
        from ktransformers_amd._native import fused_add_rmsnorm, rmsnorm

        w, eps = self.orig_module.weight, self.orig_module.variance_epsilon
        if batch_size_tensor is None:
            return rmsnorm(x, w, eps, native_rounding=True)
        if residual is not None:
            fused_add_rmsnorm(x, residual, w, eps, batch_size_tensor)
            return x, residual
        return rmsnorm(x, w, eps, native_rounding=False, bsz_tensor=batch_size_tensor)


KQwen2MoeRMSNorm = KQwen3MoeRMSNorm = DeepseekV3RMSNorm = RMSNorm


class KResidualRMSNorm(BaseInjectedModule):
    """RMS norm of an fp32 residual stream: y / sqrt(mean(y^2) + eps) * w, or * (1 + w) for weights stored around zero (`one_plus`),
    applied to a SUBLAYER'S OUTPUT and added into the residual in the same launch (post-norm decoders: x += norm(f(x))), or written
    out in the compute type (the model's last norm, with an optional row gather so that only the wanted positions reach the head).
    include/ktx_seq.h `ktx_rms_combine`.  The checkpoint tensor is the module's key itself (no `.weight` suffix) unless
    `weight_suffix` says otherwise."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 one_plus: bool | None = None, weight_suffix: str = "", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "eps", float(orig_module.eps))
        object.__setattr__(self, "one_plus", bool(orig_module.one_plus if one_plus is None else one_plus))
        object.__setattr__(self, "weight_suffix", weight_suffix)
        object.__setattr__(self, "weight_f32", None)

    def load(self):
        import torch
        w = self.gguf_loader.load_tensor(self.key + self.weight_suffix, device=torch.device(self.device))
        object.__setattr__(self, "weight_f32", w.to(torch.float32).contiguous())

    def forward(self, y, residual=None, rows=None, out_dtype=None):
        import torch
        from ktransformers_amd._native_seq import rms_combine
        return rms_combine(y, self.weight_f32, self.eps, one_plus=self.one_plus, residual=residual, rows=rows,
                           out_dtype=out_dtype or torch.float32)


class KLayerNormBias(BaseInjectedModule):
    """Layer norm with weight and bias over an fp32 residual stream: (x - mean) / sqrt(var + eps) * w + b, var = the mean of the squared
    deviations.  Two uses, one operator (include/ktx_hyb.h):

    * in FRONT of a sublayer (`forward(x)`), or as the model's last norm with a row gather (`rows=`): the normed rows in the compute
      type (`ktx_layer_norm`);
    * BEHIND a sublayer (`gated_add(x, y, ...)`): x += norm(z), z = the sublayer's result — optionally plus its output bias and plus the
      weighted rows of a mixture of experts — times sigmoid(gate logits + gate bias) when a gate is given; one launch
      (`ktx_gated_norm_add`).  With `next_norm=` (another KLayerNormBias: the pre-norm of the sublayer that follows) the same launch
      also writes that norm of the updated rows, and the call returns (x, h).

    Checkpoint tensors: the module's key (weight) and `<key>.b` (bias, optional)."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 bias_suffix: str = ".b", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "eps", float(orig_module.eps))
        object.__setattr__(self, "bias_suffix", bias_suffix)
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", None))
        object.__setattr__(self, "weight_f32", None)
        object.__setattr__(self, "bias_f32", None)

    def load(self):
        import torch
        dev = torch.device(self.device)
        object.__setattr__(self, "weight_f32", self.gguf_loader.load_tensor(self.key, device=dev).to(torch.float32).contiguous())
        if self.gguf_loader.has_tensor(self.key + self.bias_suffix):
            object.__setattr__(self, "bias_f32",
                               self.gguf_loader.load_tensor(self.key + self.bias_suffix, device=dev).to(torch.float32).contiguous())

    def forward(self, x, rows=None, out_dtype=None):
        import torch
        from ktransformers_amd._native_hyb import layer_norm
        return layer_norm(x, self.weight_f32, self.bias_f32, self.eps, rows=rows, out_dtype=out_dtype or self.compute_dtype or torch.float32)

    def post_mix(self, x_in, x_out, y=None, ybias=None, alpha: float = 1.0, stack=None, level: int = 0, depth=None, lp_dtype=None):
        """BEHIND a sublayer of a post-normed decoder whose residual is scaled: x_out = norm(alpha * x_in + y + ybias), one launch
        (`ktx_postnorm_mix`).  With `stack` (fp32 [levels, T, W]: the embedding output and every layer's result so far) the normed rows
        become level `level`, and with `depth` (a KDepthAverage) x_out is the weighted sum of levels 0 .. level instead — what a
        depth-weighted average hands to the next layer.  Returns what the following products read: x_out itself, or its copy in lp_dtype."""
        from ktransformers_amd._native_hyb import postnorm_mix
        return postnorm_mix(x_in, x_out, self.weight_f32, self.bias_f32, self.eps, alpha=alpha, y=y, ybias=ybias, stack=stack, level=level,
                            dwa=None if depth is None else depth.weights(level + 1), lp_dtype=lp_dtype)

    def gated_add(self, x, y=None, ybias=None, gate_logits=None, gate_bias=None, expert_rows=None, pair_pos=None, topk_w=None, next_norm=None):
        import torch
        from ktransformers_amd._native_hyb import gated_norm_add
        nn_ = None if next_norm is None else (next_norm.weight_f32, next_norm.bias_f32, next_norm.eps, next_norm.compute_dtype or torch.float32)
        return gated_norm_add(x, self.weight_f32, self.bias_f32, self.eps, y=y, ybias=ybias, gate_logits=gate_logits, gate_bias=gate_bias,
                              expert_rows=expert_rows, pair_pos=pair_pos, topk_w=topk_w, next_norm=nn_)


class KDepthAverage(BaseInjectedModule):
    """The weights of a depth-weighted average: behind layer i the residual handed on is sum_{j <= i + 1} w[j] X_j over the embedding
    output X_0 and the layers' results X_1 .. X_(i+1).  The sum itself runs in the launch of the layer's last norm
    (KLayerNormBias.post_mix).  Checkpoint tensor: the module's key, fp32 [i + 2]."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "w_f32", None)

    def load(self):
        import torch
        w = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(torch.float32).reshape(-1).contiguous()
        object.__setattr__(self, "w_f32", w)

    def weights(self, n: int):
        if self.w_f32.numel() != n:
            raise ValueError(f"{self.key}: an average over {n} levels takes {n} weights, the checkpoint has {self.w_f32.numel()}")
        return self.w_f32


class KScalarRMSNorm(BaseInjectedModule):
    """RMS norm whose weight is ONE number for all coordinates, over an fp32 residual stream: x * g / sqrt(mean(x^2) + eps).  It is
    also the place where what the sublayers before it produced joins the residual: one launch (include/ktx_swa.h `ktx_resid_norm`)
    adds a sublayer's output (optionally unit-RMS-normed with a weight vector first) and a mixture's weighted expert rows to x, norms
    the updated rows and — when a causal input convolution follows (`conv=`, operators/conv.py KInputConv) — lays them out with each
    request's convolution state in front, which `ktx_input_conv` then turns into what the sublayer reads; a step in which every request
    brings one token (decode) does the convolution in the norm's own launch.  `rows=` gathers rows (the model's last norm).  Checkpoint tensor: the module's key (a 0-d or 1-element tensor)."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "eps", float(orig_module.eps))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", None))
        object.__setattr__(self, "g", None)

    def load(self):
        import torch
        g = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(torch.float32).reshape(-1).contiguous()
        if g.numel() != 1:
            raise ValueError(f"{self.key}: a scalar-weight norm takes one number, got {g.numel()}")
        object.__setattr__(self, "g", g)

    def forward(self, x, batch=None, conv=None, conv_state=None, y=None, y_norm=None, moe=None, rows=None, out_dtype=None):
        """x fp32 [T, W] (+= y, moe, in place) -> the normed rows (through `conv` when given) in out_dtype."""
        import torch
        from ktransformers_amd._native_swa import FUSED_CONV_MAX_TAPS, input_conv, resid_norm
        dt = out_dtype or self.compute_dtype or torch.float32
        if conv is None or conv.taps < 1:
            return resid_norm(x, y=y, y_norm=y_norm, moe=moe, norm=(self.g, self.eps), rows=rows, out_dtype=dt)
        if conv.taps == 1 or (batch.max_q_len == 1 and conv.taps <= FUSED_CONV_MAX_TAPS):      # no neighbours, or decode steps: one launch
            return resid_norm(x, y=y, y_norm=y_norm, moe=moe, norm=(self.g, self.eps), conv=(conv.weight_f32, batch, conv_state), out_dtype=dt)
        hx = resid_norm(x, y=y, y_norm=y_norm, moe=moe, norm=(self.g, self.eps), halo=(conv.taps - 1, batch, conv_state))
        return input_conv(hx, conv.weight_f32, batch, conv_state, out_dtype=dt)


def residual_add(x, y=None, y_norm=None, moe=None):
    """x fp32 [T, W] += y (unit-RMS-normed with y_norm = (weight, eps) first when given) + a mixture's weighted expert rows, in place
    (`ktx_resid_norm` without its norm)."""
    from ktransformers_amd._native_swa import resid_norm
    if y is not None or moe is not None:
        resid_norm(x, y=y, y_norm=y_norm, moe=moe)
    return x
