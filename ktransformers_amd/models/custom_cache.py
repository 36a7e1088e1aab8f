"""Paged latent KV cache for MLA — mirror of the MLA branch of archive/ktransformers/models/custom_cache.py:26-215
(StaticCache): one `[max_pages, page_size, 1, kv_lora_rank + qk_rope_head_dim]` bf16 tensor per layer, pages of 64
tokens, an identity page table, `update()` scatters the new `[ckv | k_pe]` rows at `cache_position`.

The scatter itself is `mla_cache_append_kernel` (csrc/ktx_mla.hip); the decode path of KDeepseekV2Attention does not even
call update(): the MLA kernel stores the new row while it reads it (ktx_mla_decode_append)."""
from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch


class StaticCache:
    def __init__(self, config, max_batch_size: int, max_cache_len: Optional[int], device, dtype=None) -> None:
        self._max_batch_size = max_batch_size
        self._max_cache_len = config.max_position_embeddings if max_cache_len is None else max_cache_len
        self.dtype = dtype if dtype is not None else torch.bfloat16
        if self.dtype != torch.bfloat16:
            raise ValueError("the HIP MLA kernels read a bf16 latent cache")
        self.page_size = 64                                                      # custom_cache.py:81
        self.max_pages = (self._max_cache_len + self.page_size - 1) // self.page_size
        self.kv_lora_rank = config.kv_lora_rank
        self.qk_rope_head_dim = config.qk_rope_head_dim
        self.num_hidden_layers = config.num_hidden_layers
        self.is_MLA, self.is_page = True, True
        self.identity_page_table = True      # page_table_list[i] = arange (custom_cache.py:99-104): pages are used in order
        latent_shape = (self.max_pages, self.page_size, 1, self.kv_lora_rank + self.qk_rope_head_dim)
        self.key_cache, self.value_cache, self.page_table_list, self.past_tokens = [], [], [], []
        self.page_table_map: Dict[Any, torch.Tensor] = {}
        for idx in range(self.num_hidden_layers):
            dev = device[f"blk.{idx}.self_attn"]["generate_device"] if isinstance(device, dict) else device
            if dev not in self.page_table_map:                                   # custom_cache.py:99-104
                pt = torch.arange(max_batch_size * self.max_pages, dtype=torch.int32, device=dev)
                self.page_table_map[dev] = pt.view(max_batch_size, self.max_pages)
            self.page_table_list.append(self.page_table_map[dev])
            self.key_cache.append(torch.zeros(latent_shape, dtype=self.dtype, device=dev))
            self.value_cache.append(None)
            self.past_tokens.append(0)

    @property
    def max_batch_size(self):
        return self._max_batch_size

    @property
    def max_cache_len(self):
        return self._max_cache_len

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """key_states = compressed_kv [.., T, 1, kv_lora], value_states = k_pe [.., T, 1, rope] (custom_cache.py:147-199)."""
        from ktransformers_amd._native import mla_cache_append

        cache_position = cache_kwargs.get("cache_position")
        k_out = self.key_cache[layer_idx]
        if self.past_tokens[layer_idx] + cache_position.size(0) > self.max_pages * self.page_size:
            # the reference's indexed assignment raises on an out-of-range position (custom_cache.py:189-195)
            raise IndexError(f"StaticCache.update: {self.past_tokens[layer_idx]} + {cache_position.size(0)} tokens exceed the "
                             f"cache ({self.max_pages * self.page_size} tokens)")
        self.past_tokens[layer_idx] += cache_position.size(0)
        page_idx = cache_position // self.page_size
        page_offset = cache_position % self.page_size
        mla_cache_append(k_out, key_states.reshape(-1, self.kv_lora_rank), value_states.reshape(-1, self.qk_rope_head_dim),
                         page_idx, page_offset)
        return k_out, self.page_table_list[layer_idx]

    def note_appended(self, layer_idx: int, n: int) -> None:
        """Bookkeeping for rows the attention kernel appended itself."""
        self.past_tokens[layer_idx] += n

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.past_tokens[layer_idx]

    def get_usable_length(self, kv_seq_len: int, layer_idx: Optional[int] = 0) -> int:
        return 0                                                                 # custom_cache.py:225-226 (callers add it to q_len)

    def change_seq_length(self, bias: Optional[int] = 0) -> None:
        for i in range(self.num_hidden_layers):
            self.past_tokens[i] += bias

    def get_max_length(self) -> Optional[int]:
        return self._max_cache_len

    def reset(self):
        for i in range(self.num_hidden_layers):
            self.key_cache[i].zero_()
            self.past_tokens[i] = 0

    def remove_suffix(self, start_pos: int) -> None:
        """Forget everything from token `start_pos` on (prefix reuse between requests, custom_cache.py:240-250)."""
        for i in range(self.num_hidden_layers):
            k = self.key_cache[i]
            k.view(-1, k.shape[-1])[start_pos:].zero_()
            self.past_tokens[i] = start_pos

    def get_max_cache_shape(self):
        return self.max_cache_len                                                # custom_cache.py:252-254


class KDeepSeekV3Cache:
    """The batched-serving latent cache (archive/ktransformers/models/custom_cache.py:387-466): per layer one
    [pages, page_size, 1, kv_lora_rank + rope] bf16 tensor, pages handed out by the scheduler.  The reference takes the tensors
    from its kvc2 `InferenceContext`; here `allocate(num_pages)` creates them (the storage engine is out of scope) and `load`
    accepts any object with the same `k_cache[0][layer]` shape of attribute."""

    def __init__(self, config, page_size: int = 256, dtype=torch.bfloat16, device="cuda:0"):
        if dtype != torch.bfloat16:
            raise ValueError("the HIP MLA kernels read a bf16 latent cache")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        self.kv_lora_rank, self.qk_rope_head_dim, self.page_size = config.kv_lora_rank, config.qk_rope_head_dim, page_size
        self.k_caches, self.v_caches = [], []
        self.max_cache_len = 0

    def allocate(self, num_pages: int) -> None:
        shape = (num_pages, self.page_size, 1, self.kv_lora_rank + self.qk_rope_head_dim)
        self.k_caches = [torch.zeros(shape, dtype=self.dtype, device=self.device) for _ in range(self.config.num_hidden_layers)]
        self.max_cache_len = num_pages * self.page_size

    def load(self, inference_context) -> None:
        self.k_caches = [inference_context.k_cache[0][i] for i in range(self.config.num_hidden_layers)]
        self.max_cache_len = self.k_caches[0].shape[0] * self.k_caches[0].shape[1]

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int, page_idx: torch.Tensor,
               page_offset: torch.Tensor, cache_kwargs: Optional[Dict[str, Any]] = None) -> torch.Tensor:
        """Scatter the new latent rows (key_states = compressed_kv, value_states = k_pe) to [page_idx, page_offset]; returns the
        layer's whole cache tensor (custom_cache.py:413-443)."""
        from ktransformers_amd._native import mla_cache_append

        k_out = self.k_caches[layer_idx]
        mla_cache_append(k_out, key_states.reshape(-1, self.kv_lora_rank), value_states.reshape(-1, self.qk_rope_head_dim),
                         page_idx, page_offset)
        return k_out

    def get_page_table(self, cache_position: torch.Tensor, q_indptr: torch.Tensor, kv_indptr: torch.Tensor, kv_indices: torch.Tensor,
                       bsz_tensors: torch.Tensor):
        """(page_idx, page_offset) of every scheduled token (custom_cache.py:446-463): token i of request r at position p lives
        in that request's p // page_size-th page, kv_indices[kv_indptr[r] + p // page_size]; tokens beyond bsz_tensors[0], and
        positions beyond the request's allotted pages, get page 0 like the reference's zero initialisation.  Vectorised: the
        reference loops over tokens on the host."""
        page_offset = cache_position % self.page_size
        local = cache_position // self.page_size
        n = cache_position.numel()
        counts = (q_indptr[1:] - q_indptr[:-1]).to(torch.long)
        query_ids = torch.repeat_interleave(torch.arange(counts.numel(), device=cache_position.device), counts, output_size=int(q_indptr[-1]))
        if query_ids.numel() < n:   # tokens past the last request keep request 0, as torch.zeros_like does in the reference
            query_ids = torch.cat([query_ids, query_ids.new_zeros(n - query_ids.numel())])
        query_ids = query_ids[:n]
        start = kv_indptr[query_ids].to(torch.long)
        have = (kv_indptr[query_ids + 1] - kv_indptr[query_ids]).to(torch.long)
        ok = (local < have) & (torch.arange(n, device=cache_position.device) < int(bsz_tensors[0]))
        idx = (start + torch.where(ok, local.to(torch.long), torch.zeros_like(start))).clamp_(max=max(kv_indices.numel() - 1, 0))
        page_idx = torch.where(ok, kv_indices[idx].to(local.dtype), torch.zeros_like(local))
        return page_idx, page_offset



class ForwardBatch:
    """What one scheduled step looks like to the sequence-mixer operators (include/ktx_seq.h): the tokens of all requests flattened,
    int32 device tensors.  positions / tok_req / cache_loc per token; q_indptr / pos0 / slot / page_indptr per request;
    page_indices = the requests' page lists back to back.  nsplit = workgroups that share one query token's keys."""
    __slots__ = ("T", "B", "positions", "tok_req", "cache_loc", "q_indptr", "pos0", "slot", "page_indptr", "page_indices",
                 "max_q_len", "max_kv_len", "nsplit")

    def __init__(self, **kw):
        for k in self.__slots__:
            setattr(self, k, kw.get(k))


class KHybridCache:
    """Cache and state manager of decoders that mix paged attention with recurrent layers.

    Per layer, whatever its spec names:
      "attn": (kv_heads, dim)  — a paged KEY cache [pages * page_size, kv_heads, dim] (bf16 or fp32) for attention whose values are its
                                 un-normed keys, plus fp32 1 / rms(k) per row and key head;
      "latent": width          — a paged cache of latent rows [pages * page_size, width] (bf16 or fp32): what a latent attention keeps
                                 per token (normed latent + rotated key part);
      "kv": (kv_heads, dim, vdim) — paged KEY rows [pages * page_size, kv_heads, dim] and VALUE rows [.., kv_heads, vdim] (bf16 or
                                 fp32) for grouped-query attention, stored as the attention reads them (rotated, normed);
      "rec": (heads, dim, vdim)   — fp32 state slots S [slots, heads, dim, vdim], n [slots, heads, dim], m [slots, heads] (mLSTM);
      "delta": (heads, dim, vdim) — fp32 state slots S alone (delta rule);
      "ssm": (channels, state)    — fp32 state slots S [slots, channels, state] (selective scan);
      "conv": (channels, taps)    — fp32 slots [slots, taps - 1, channels]: the inputs a short causal convolution still needs;
      "pre": [(channels, taps), ...] — the same kind of slots for convolutions on what the layer's sublayers read, one per sublayer
                                 (an entry with taps <= 1 or None holds nothing).
    A layer that runs several times with the same weights (a repeated block) has one spec, and so one cache or state, per run.
    A request holds a list of pages (grown as it grows) and one slot from admit() to release(); freed pages and slots go back on
    LIFO free lists and are handed out again without being cleared: the attention kernels never read past a request's length and
    the recurrences start from zero at position 0 whatever the slot holds.

    plan() turns (request, n new tokens) pairs into a ForwardBatch; the operators append and read through it."""

    def __init__(self, layer_specs, max_tokens: int, max_requests: int = 8, page_size: int = 64, dtype=torch.bfloat16,
                 device="cuda:0"):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("KHybridCache: bf16 or fp32 key cache")
        self.layer_specs, self.page_size, self.dtype, self.device = list(layer_specs), int(page_size), dtype, torch.device(device)
        self.max_requests = int(max_requests)
        # every live request may leave one page partly filled
        self.num_pages = (int(max_tokens) + self.page_size - 1) // self.page_size + self.max_requests
        self.max_cache_len = self.num_pages * self.page_size
        rows = self.num_pages * self.page_size
        self.k_caches, self.k_inv, self.S, self.n, self.m, self.lat_caches, self.conv = [], [], [], [], [], [], []
        self.v_caches, self.pre_conv = [], []
        for spec in self.layer_specs:
            a, r, lat, dl, cv = spec.get("attn"), spec.get("rec"), spec.get("latent"), spec.get("delta"), spec.get("conv")
            kv, ssm = spec.get("kv"), spec.get("ssm")
            if sum(1 for s_ in (r, dl, ssm) if s_) > 1:
                raise ValueError("KHybridCache: a layer run has one recurrent state (\"rec\", \"delta\" or \"ssm\")")
            if a and kv:
                raise ValueError("KHybridCache: a layer run has one key cache (\"attn\" or \"kv\")")
            self.v_caches.append(torch.zeros((rows, kv[0], kv[2]), dtype=dtype, device=self.device) if kv else None)
            self.pre_conv.append([torch.zeros((self.max_requests, pc[1] - 1, pc[0]), dtype=torch.float32, device=self.device)
                                  if pc and pc[1] > 1 else None for pc in (spec.get("pre") or [])])
            if kv:
                a = (kv[0], kv[1])
            self.k_caches.append(torch.zeros((rows, a[0], a[1]), dtype=dtype, device=self.device) if a else None)
            a = spec.get("attn")
            self.k_inv.append(torch.zeros((rows, a[0]), dtype=torch.float32, device=self.device) if a else None)
            self.lat_caches.append(torch.zeros((rows, int(lat)), dtype=dtype, device=self.device) if lat else None)
            self.conv.append(torch.zeros((self.max_requests, cv[1] - 1, cv[0]), dtype=torch.float32, device=self.device)
                             if cv and cv[1] > 1 else None)
            r = r or dl or ssm
            self.S.append(torch.zeros((self.max_requests,) + tuple(r), dtype=torch.float32, device=self.device) if r else None)
            r = spec.get("rec")
            self.n.append(torch.zeros((self.max_requests, r[0], r[1]), dtype=torch.float32, device=self.device) if r else None)
            self.m.append(torch.zeros((self.max_requests, r[0]), dtype=torch.float32, device=self.device) if r else None)
        self.free_pages = list(range(self.num_pages - 1, -1, -1))
        self.free_slots = list(range(self.max_requests - 1, -1, -1))
        self.requests: Dict[Any, dict] = {}
        self.generation = 0          # bumped whenever the tensors are re-allocated (captured graphs hold their addresses)

    # ---- allocation ------------------------------------------------------------------------------------------------
    def admit(self, rid) -> None:
        if rid in self.requests:
            raise KeyError(f"KHybridCache: request {rid!r} is already live")
        if not self.free_slots:
            self._add_slots(self.max_requests)
        self.requests[rid] = {"pages": [], "len": 0, "slot": self.free_slots.pop()}

    def release(self, rid) -> None:
        r = self.requests.pop(rid)
        self.free_pages.extend(reversed(r["pages"]))
        self.free_slots.append(r["slot"])

    def seq_len(self, rid) -> int:
        return self.requests[rid]["len"]

    def state_tensors(self) -> list:
        """Every per-slot tensor a step advances in place (what a caller saves around runs that must not count)."""
        return [t for group in (self.S, self.n, self.m, self.conv) for t in group if t is not None] + \
            [t for group in self.pre_conv for t in group if t is not None]

    def live_tokens(self) -> int:
        return sum(r["len"] for r in self.requests.values())

    def _grow(self, r: dict, n_new: int) -> None:
        need = (r["len"] + n_new + self.page_size - 1) // self.page_size - len(r["pages"])
        if need > len(self.free_pages):
            self._add_pages(max(need - len(self.free_pages), self.num_pages // 2))
        for _ in range(max(need, 0)):
            r["pages"].append(self.free_pages.pop())

    # The cache is sized by the caller's estimate (tokens and requests live at a time); a step that needs more gets it: the tensors are
    # re-allocated with the old contents in front (new page / slot numbers follow the old ones), which invalidates captured graphs
    # — the single-request view below reserves everything up front and never grows.
    def _add_slots(self, extra: int) -> None:
        grow = lambda t: None if t is None else torch.cat([t, torch.zeros((extra,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)])
        self.S, self.n, self.m = [grow(t) for t in self.S], [grow(t) for t in self.n], [grow(t) for t in self.m]
        self.conv = [grow(t) for t in self.conv]
        self.pre_conv = [[grow(t) for t in group] for group in self.pre_conv]
        self.free_slots.extend(range(self.max_requests + extra - 1, self.max_requests - 1, -1))
        self.max_requests += extra
        self.generation += 1

    def _add_pages(self, extra: int) -> None:
        rows = extra * self.page_size
        grow = lambda t: None if t is None else torch.cat([t, torch.zeros((rows,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)])
        self.k_caches, self.k_inv = [grow(t) for t in self.k_caches], [grow(t) for t in self.k_inv]
        self.lat_caches = [grow(t) for t in self.lat_caches]
        self.v_caches = [grow(t) for t in self.v_caches]
        self.free_pages.extend(range(self.num_pages + extra - 1, self.num_pages - 1, -1))
        self.num_pages += extra
        self.max_cache_len = self.num_pages * self.page_size
        self.generation += 1

    def plan_lists(self, entries) -> dict:
        """The host half of plan(): grows each request's page list, advances its length and returns the step's metadata as python
        lists (same field names as ForwardBatch) — what a captured decode graph copies into its static buffers."""
        ps = self.page_size
        d = {k: [] for k in ("positions", "tok_req", "cache_loc", "pos0", "slot", "page_indices")}
        d["q_indptr"], d["page_indptr"] = [0], [0]
        max_q = max_kv = 0
        for b, (rid, n_new) in enumerate(entries):
            r = self.requests[rid]
            self._grow(r, n_new)
            start, pages = r["len"], r["pages"]
            for p in range(start, start + n_new):
                d["positions"].append(p)
                d["tok_req"].append(b)
                d["cache_loc"].append(pages[p // ps] * ps + p % ps)
            r["len"] = start + n_new
            d["q_indptr"].append(d["q_indptr"][-1] + n_new)
            d["pos0"].append(start)
            d["slot"].append(r["slot"])
            d["page_indices"].extend(pages)
            d["page_indptr"].append(len(d["page_indices"]))
            max_q, max_kv = max(max_q, n_new), max(max_kv, r["len"])
        d.update(T=len(d["positions"]), B=len(entries), max_q_len=max_q, max_kv_len=max_kv)
        return d

    def plan(self, entries, target_workgroups: int = 1024, keys_per_split: int = 128) -> ForwardBatch:
        """entries: [(request id, number of new tokens)], in batch order -> the step's ForwardBatch (plan_lists on the device)."""
        d = self.plan_lists(entries)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=self.device)
        nsplit = max(1, min(target_workgroups // max(d["T"], 1), (d["max_kv_len"] + keys_per_split - 1) // keys_per_split))
        return ForwardBatch(T=d["T"], B=d["B"], max_q_len=d["max_q_len"], max_kv_len=d["max_kv_len"], nsplit=nsplit,
                            **{k: i32(d[k]) for k in ("positions", "tok_req", "cache_loc", "q_indptr", "pos0", "slot", "page_indptr",
                                                      "page_indices")})

    # ---- the single-request view util.generate.prefill_and_generate drives (one sequence, positions given by the caller) --------
    SINGLE = "__single__"

    def single_request_batch(self, position_ids: torch.Tensor) -> ForwardBatch:
        """A ForwardBatch for ONE implicit request whose new tokens sit at `position_ids` ([T] or [1, T], consecutive).  All pages
        the cache has are reserved for it at the first call, so a one-token step needs no host knowledge of the position: every
        tensor is derived from position_ids on the device and a captured graph of the step stays valid as the sequence grows."""
        ps = self.page_size
        if self.SINGLE not in self.requests:
            self.admit(self.SINGLE)
            r = self.requests[self.SINGLE]
            r["pages"] = [self.free_pages.pop() for _ in range(len(self.free_pages))]
            r["page_t"] = torch.tensor(r["pages"], dtype=torch.int32, device=self.device)
            r["slot_t"] = torch.tensor([r["slot"]], dtype=torch.int32, device=self.device)
            r["page_indptr"] = torch.tensor([0, len(r["pages"])], dtype=torch.int32, device=self.device)
            r["q_indptr1"] = torch.tensor([0, 1], dtype=torch.int32, device=self.device)
            r["tok_req1"] = torch.zeros(1, dtype=torch.int32, device=self.device)
        r = self.requests[self.SINGLE]
        pos = position_ids.reshape(-1).to(device=self.device, dtype=torch.int32)
        T = pos.numel()
        loc = (r["page_t"][(pos // ps).long()] * ps + pos % ps).int()
        cap = len(r["pages"]) * ps
        one = T == 1     # (a one-token step allocates nothing on the host: it may be captured into a graph)
        return ForwardBatch(T=T, B=1, positions=pos, cache_loc=loc, pos0=pos[:1],
                            tok_req=r["tok_req1"] if one else torch.zeros(T, dtype=torch.int32, device=self.device),
                            q_indptr=r["q_indptr1"] if one else torch.tensor([0, T], dtype=torch.int32, device=self.device),
                            slot=r["slot_t"], page_indptr=r["page_indptr"], page_indices=r["page_t"], max_q_len=T, max_kv_len=cap,
                            nsplit=max(1, min(1024, (cap + 127) // 128)) if one else 1)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        r = self.requests.get(self.SINGLE)
        return r["len"] if r else 0

    def get_max_length(self) -> Optional[int]:
        return self.max_cache_len

    def reset(self) -> None:
        for rid in list(self.requests):
            self.release(rid)
