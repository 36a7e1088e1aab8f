"""Softmax-routed mixture of relu^2 experts with identity experts on an fp32 residual stream, any sizes, bf16 or fp32 — an injected
operator beside operators/sigmoid_moe.py (sigmoid scores, GLU experts) and the quantised MoE operators (experts.py, gate.py):

    s = softmax(W_router h) over ALL router outputs (fp32);  the `top` outputs with the largest s + correction are chosen;  their
    weights are s (without the correction) over (the chosen s' sum + 1e-20);  expert e: W_down relu(W_up h)^2, no biases;  the LAST
    `identity` router outputs stand for experts without weights that return h itself.

The real experts run as two grouped products over the (token, choice) pairs sorted by router output (include/ktx_hyb.h `ktx_moe_plan`; small
steps route and sort in one launch, `ktx_softmax_route_plan`;
`ktx_grouped_gemm` / `ktx_grouped_gemv` with the relu^2 epilogue; groups beyond the real experts are skipped); the weighted sum over a
token's choices — rows of real experts, h for identity ones — is left to the consumer's launch (`ktx_resid_norm`), so forward returns the
pieces.  top, identity and the sum's eps are constructor arguments (read from the replaced module).  Checkpoint tensors:
`<key>.router` [experts + identity, width], `<key>.correction` [experts + identity] (optional), `<key>.e<i>.{up,down}`."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KSoftmaxRoutedMoE(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        for name in ("experts", "identity", "top", "sum_eps", "ff", "width"):
            object.__setattr__(self, name, getattr(orig_module, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        get = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(cd)
        E, F, W, R = self.experts, self.ff, self.width, self.experts + self.identity
        self.w["router"] = get("router").contiguous()
        self.w["correction"] = ld.load_tensor(f"{self.key}.correction", device=dev).to(torch.float32).contiguous() \
            if ld.has_tensor(f"{self.key}.correction") else None
        self.w["up"] = torch.stack([get(f"e{e}.up") for e in range(E)]).contiguous()
        self.w["down"] = torch.stack([get(f"e{e}.down") for e in range(E)]).contiguous()
        if tuple(self.w["up"].shape) != (E, F, W) or tuple(self.w["down"].shape) != (E, W, F) or tuple(self.w["router"].shape) != (R, W) or \
                (self.w["correction"] is not None and self.w["correction"].numel() != R):
            raise ValueError(f"{self.key}: tensors do not fit experts={E} identity={self.identity} ff={F} width={W}")

    def forward(self, h: torch.Tensor):
        """h [T, width] in the compute type -> the pieces of the weighted sum: (expert_rows fp32 [T * top, width] in sorted order,
        pair_pos int32 [T * top], topk_idx int32 [T, top], topk_w fp32 [T, top], number of real experts, h)."""
        from ktransformers_amd._native_hyb import WIDE_MIN_ROWS_PER_EXPERT, expert_gemm, moe_plan
        from ktransformers_amd._native_seq import dense_gemm_skinny
        from ktransformers_amd._native_swa import ROUTE_PLAN_MAX_T, softmax_route, softmax_route_plan
        E, R = self.experts, self.experts + self.identity
        logits = dense_gemm_skinny(h, self.w["router"])
        if h.shape[0] <= ROUTE_PLAN_MAX_T:       # decode steps: router and sort in one launch
            idx, wts, plan = softmax_route_plan(logits, self.top, self.sum_eps, self.w["correction"])
        else:
            idx, wts = softmax_route(logits, self.top, self.sum_eps, self.w["correction"])
            wide = self.compute_dtype == torch.bfloat16 and h.shape[0] * self.top >= WIDE_MIN_ROWS_PER_EXPERT * R
            plan = moe_plan(idx, R, wide=wide)
        act = expert_gemm(h, self.w["up"], plan, gather=True, out_dtype=self.compute_dtype, act="relu_sq")
        rows = expert_gemm(act, self.w["down"], plan, gather=False)
        return rows, plan.pair_pos, idx, wts, E, h
