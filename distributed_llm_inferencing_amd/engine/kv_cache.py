"""Paged KV cache storage for one pipeline stage (its layers only).

Two tensors per stage (one allocation each, sized from free HBM):
    K: [L_stage, num_blocks, Hkv, block_size, hd]
    V: [L_stage, num_blocks, Hkv, block_size, hd]   (token-major like K, see ops/reference.py)
Zero-initialised once so rows past a sequence's context are always finite (the decode
kernel reads whole 32-token tiles and multiplies the masked ones by 0).
"""
from __future__ import annotations

import os
from typing import List, Optional, Tuple

import torch

from ..models.configs import ModelConfig


def bytes_per_block(cfg: ModelConfig, num_layers: int, block_size: int, dtype_bytes: int = 2):
    if cfg.is_hybrid:
        return max(1, cfg.kv_bytes_per_token(dtype_bytes)) * block_size
    return 2 * num_layers * cfg.num_kv_heads * cfg.head_dim * block_size * dtype_bytes


def blocks_for_budget(cfg: ModelConfig, num_layers: int, block_size: int, budget_bytes: int):
    return max(1, int(budget_bytes // max(1, bytes_per_block(cfg, num_layers, block_size))))


def auto_num_blocks(cfg: ModelConfig, num_layers: int, block_size: int, device,
                    fraction: float = 0.85, reserve_bytes: Optional[int] = None,
                    cap_tokens: int = 0, pending_bytes: int = 0) -> int:
    """Blocks that fit in ``fraction`` of the HBM still free (weights already resident)
    minus a reserve for activations, GEMM workspaces and graph pools: the KV pool is sized
    for the 288 GB of an MI355X (Llama-3-8B: ~1.7M tokens of context on one GPU), not for
    max_batch x max_model_len. ``cap_tokens`` / ``DLI_KV_MAX_TOKENS`` cap it (0 = no cap).
    ``pending_bytes``: weights that will land on this device after the pool is sized (a
    pipeline stage sizes its pool before it loads its layers; ranks sharing one device pass
    every rank's). Ranks sharing one device (``DLI_SAME_DEVICE=1`` rehearsals) split the rest
    by ``LOCAL_WORLD_SIZE``."""
    dev = torch.device(device)
    env_cap = int(os.environ.get("DLI_KV_MAX_TOKENS", "0") or 0)
    cap_tokens = env_cap or cap_tokens
    if dev.type == "cuda":
        free, total = torch.cuda.mem_get_info(dev)
        free = max(0, free - int(pending_bytes))
        if reserve_bytes is None:
            reserve_bytes = max(8 << 30, int(0.03 * total))
        if os.environ.get("DLI_SAME_DEVICE", "0") == "1":
            ranks = os.environ.get("LOCAL_WORLD_SIZE", os.environ.get("WORLD_SIZE"))
            if ranks is None:
                # a worker that joined a ring by init_method (no launcher environment)
                import torch.distributed as dist
                ranks = dist.get_world_size() if dist.is_initialized() else 1
            fraction /= max(1, int(ranks))
        budget = max(0, int(free * fraction) - reserve_bytes)
    else:
        budget = 256 << 20                  # CPU (tests / the gpt2 plumbing config)
        cap_tokens = cap_tokens or (1 << 16)
    n = blocks_for_budget(cfg, max(1, num_layers), block_size, budget)
    if cap_tokens:
        n = min(n, -(-cap_tokens // block_size))
    return max(n, 16)


class KVCache:
    def __init__(self, cfg: ModelConfig, num_layers: int, num_blocks: int, block_size: int,
                 device, dtype=torch.bfloat16):
        self.cfg = cfg
        self.num_layers = num_layers
        self.num_blocks = num_blocks
        self.block_size = block_size
        hkv, hd = cfg.num_kv_heads, cfg.head_dim
        self.k = torch.zeros(num_layers, num_blocks, hkv, block_size, hd, dtype=dtype, device=device)
        self.v = torch.zeros(num_layers, num_blocks, hkv, block_size, hd, dtype=dtype, device=device)

    def layers(self) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        return [(self.k[i], self.v[i]) for i in range(self.num_layers)]

    @property
    def nbytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()

    @property
    def capacity_tokens(self) -> int:
        return self.num_blocks * self.block_size


class HybridCache:
    """Caches and recurrent states of a hybrid design, one entry per layer run (a looped layer
    has one per pass), all addressed by the engine's one block manager / state-slot manager:

    * ``attention``:        (k [slots, G*d], v [slots, G*d])   token-major rows, slot =
                            block * block_size + offset; k holds the normed keys, v the raw ones
    * ``latent_attention``: (c [slots, kv_rank + rot_dim],)     normed latent | rotated key; a
                            layer with ``kv_from`` gets that layer's tensor (it writes nothing)
    * ``hgrn2``, ``gla``:   (state [state_slots, H, d, dv] fp32,)  one slot per live sequence
    * ``talk_attention``:   (k [slots, G*d], v [slots, G*dv])   normed keys and values; a layer
                            with ``kv_from`` gets the tensors of that layer's run (it writes
                            nothing)

    * ``lightning``:        (state [state_slots, H, d, dv] fp32,)
    * ``parallel``:         (k [slots, G*d], v [slots, G*dv], state [state_slots, Hr, dr, dvr]
                            fp32, nm [state_slots, Hr, dr + 1] fp32): the attention side's
                            normed, rotated keys and values; the memory side's matrix, and its
                            normaliser vector followed by its running maximum

    ``shift_states[run]`` is [state_slots, D] fp32 for a layer with token shift (the previous
    token's mixer input), else None. ``prev_token`` is int32 [state_slots] for a design whose
    embedding reads the previous token (hashed bigrams), else None.

    Rows are zero-initialised once (padding rows of captured decode steps read row 0). A state
    slot is not cleared on reuse: a sequence's first portion starts from zero by position."""

    def __init__(self, cfg: ModelConfig, num_blocks: int, block_size: int, state_slots: int,
                 device, dtype=torch.bfloat16):
        self.cfg = cfg
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.state_slots = state_slots
        self.num_layers = len(cfg.layer_runs())
        rows = num_blocks * block_size
        self.entries = []
        self.shift_states = []
        self.prev_token = (torch.zeros(state_slots, dtype=torch.int32, device=device)
                           if cfg.bigram else None)
        run_of = {}                       # layer -> its (last) run, for layers that lend their cache
        for ri, (li, _, _) in enumerate(cfg.layer_runs()):
            s = cfg.layer_specs[li]
            self.shift_states.append(
                torch.zeros(state_slots, cfg.hidden_size, dtype=torch.float32, device=device)
                if s.shift else None)
            if s.kind == "latent_attention" and s.kv_from >= 0:
                self.entries.append(self.entries[run_of[s.kv_from]])
                run_of[li] = ri
                continue
            if s.kind == "talk_attention":
                if s.kv_from >= 0:
                    e = self.entries[run_of[s.kv_from]]
                else:
                    e = (torch.zeros(rows, s.kv_heads * s.dim, dtype=dtype, device=device),
                         torch.zeros(rows, s.kv_heads * s.vdim, dtype=dtype, device=device))
                run_of[li] = ri
                self.entries.append(e)
                continue
            run_of[li] = ri
            if s.kind == "attention":
                e = (torch.zeros(rows, s.kv_heads * s.dim, dtype=dtype, device=device),
                     torch.zeros(rows, s.kv_heads * s.dim, dtype=dtype, device=device))
            elif s.kind == "latent_attention":
                e = (torch.zeros(rows, s.kv_rank + s.rot_dim, dtype=dtype, device=device),)
            elif s.kind == "parallel":
                l, r = s.left, s.right
                e = (torch.zeros(rows, l.kv_heads * l.dim, dtype=dtype, device=device),
                     torch.zeros(rows, l.kv_heads * l.vdim, dtype=dtype, device=device),
                     torch.zeros(state_slots, r.heads, r.dim, r.vdim, dtype=torch.float32,
                                 device=device),
                     torch.zeros(state_slots, r.heads, r.dim + 1, dtype=torch.float32,
                                 device=device))
            else:
                e = (torch.zeros(state_slots, s.heads, s.dim, s.vdim, dtype=torch.float32,
                                 device=device),)
            self.entries.append(e)

    def layers(self) -> "HybridCache":
        """What the runner hands to the model: the cache itself (entries + block size)."""
        return self

    @property
    def nbytes(self) -> int:
        own = {t.data_ptr(): t for e in self.entries for t in e}
        own.update({t.data_ptr(): t for t in self.shift_states if t is not None})
        return sum(t.numel() * t.element_size() for t in own.values())

    @property
    def capacity_tokens(self) -> int:
        return self.num_blocks * self.block_size


class StateSlots:
    """Recurrent-state slots of the live sequences: a free list over ``num_slots`` rows of the
    state tensors (``HybridCache``). A sequence takes a slot when it is admitted and gives it
    back when it finishes or is preempted; slots are reused without clearing."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._of: dict = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def get(self, seq_id: int) -> int:
        return self._of.get(seq_id, -1)

    def acquire(self, seq_id: int) -> int:
        s = self._of.get(seq_id)
        if s is None:
            if not self._free:
                return -1
            s = self._of[seq_id] = self._free.pop()
        return s

    def release(self, seq_id: int) -> None:
        s = self._of.pop(seq_id, None)
        if s is not None:
            self._free.append(s)
