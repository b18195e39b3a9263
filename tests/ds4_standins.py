"""Torch stand-ins for the third-party DS4 attention block and cache that the layer wrappers wrap.

Reduced hidden sizes with the real head geometry, after the reference's _build_synthetic_attention and
_make_steady_cache (tests/test_deepseek_v4_decode_attention_kernel.py:376-445). Only what the wrappers
touch exists: projections, norms, a compressor that returns the pool a test put into the cache state, a
ring cache with the steady-state fields.
"""

from types import SimpleNamespace

import numpy as np
import torch

from oracle import ds4

OFFSET = 3855
_YARN = {"factor": 16.0, "original_seq_len": 65536, "beta_fast": 32, "beta_slow": 1}


class Rope:
    dims = 64

    def __init__(self, base, yarn, device):
        self.inv_freq = torch.from_numpy(ds4.rope_inverse_frequencies(64, base, yarn).astype(np.float32)).to(device)


class Ring:
    """Steady-state fields of the rotating local cache."""

    def __init__(self, keys, offset, idx):
        self.keys = keys
        self.values = keys.clone()
        self.offset = offset
        self._idx = idx
        self.max_size = int(keys.shape[2])
        self.keep = 0


class _CacheBase:
    def __init__(self, ring):
        self.local = ring
        self.compressor_state = {}
        self.indexer_state = {}
        self.update_calls = 0
        self.trim_calls = 0

    @property
    def offset(self):
        return self.local.offset

    def update_and_fetch(self, keys, values):
        self.update_calls += 1
        self.last_update = (keys, values)
        return keys, values

    def trim(self, n):
        self.trim_calls += 1
        return n


class Cache(_CacheBase):
    """The cache class the wrappers are installed for."""


class OtherCache(_CacheBase):
    """Same fields, another class: wrappers must not engage on it."""


class Compressor:
    """Returns the pool held in the cache state (the steady-state token appends no pool row) and, like the
    real one, keeps state per token: every call is recorded with its position and counted in the cache
    state, so a token that advances it twice shows."""

    def __init__(self):
        self.calls = []
        self.positions = []

    def __call__(self, x, rope, cache, offset, state_key="compressor_state"):
        self.calls.append(state_key)
        self.positions.append(int(offset))
        state = getattr(cache, state_key)
        state["advances"] = state.get("advances", 0) + 1
        return state["pooled"]


class Indexer:
    def __init__(self, hidden, q_lora, n_heads, topk, device, gen):
        self.n_heads, self.head_dim, self.index_topk = n_heads, 128, topk
        self.scale = 128 ** -0.5
        self.compressor = Compressor()
        self.wq_b = _linear(q_lora, n_heads * 128, device, gen)
        self.weights_proj = _linear(hidden, n_heads, device, gen)
        self.stock_calls = 0

    def __call__(self, x, q_residual, rope, position_rope, cache, start_pos):
        # the stock indexer advances its compressor itself
        self.stock_calls += 1
        self.compressor(x, rope, cache, start_pos, state_key="indexer_state")
        return None


def _linear(n_in, n_out, device, gen):
    lin = torch.nn.Linear(n_in, n_out, bias=False, device=device, dtype=torch.float16)
    with torch.no_grad():
        lin.weight.copy_((torch.randn((n_out, n_in), generator=gen) * n_in ** -0.5).to(torch.float16))
    return lin


class Attention:
    """The attention block the fused decode wrapper wraps (stock path = recorded calls only)."""

    compress_ratio = 4
    head_dim = 512

    def __init__(self, device, *, hidden=256, n_heads=8, q_lora=64, index_heads=8, topk=64, seed=11):
        gen = torch.Generator().manual_seed(seed)
        self.args = SimpleNamespace(sliding_window=128, rms_norm_eps=1e-6, hidden_size=hidden)
        self.n_heads = n_heads
        self.rope = Rope(10000.0, None, device)
        self.compress_rope = Rope(160000.0, _YARN, device)
        self.wq_a = _linear(hidden, q_lora, device, gen)
        self.q_norm = torch.nn.RMSNorm(q_lora, eps=1e-6, device=device, dtype=torch.float16)
        self.wq_b = _linear(q_lora, n_heads * 512, device, gen)
        self.wkv = _linear(hidden, 512, device, gen)
        self.kv_norm = torch.nn.RMSNorm(512, eps=1e-6, device=device, dtype=torch.float16)
        self.compressor = Compressor()
        self.indexer = Indexer(hidden, q_lora, index_heads, topk, device, gen)
        self.attn_sink = (torch.randn((n_heads,), generator=gen) * 0.3).to(device)
        self.softmax_scale = 512 ** -0.5
        self.wo_b = _linear(n_heads * 512, hidden, device, gen)
        self.stock_calls = []
        self.tail_calls = []
        self.heads_seen = None

    def _grouped_output_projection(self, out):
        self.heads_seen = out
        return out

    def __call__(self, x, mask=None, cache=None):
        self.stock_calls.append((tuple(x.shape), cache))
        return x

    def composed_decode_tail(self, **kwargs):
        self.tail_calls.append(kwargs)
        return kwargs["x"]


def steady_cache(device, *, rows, offset=OFFSET, idx=37, cls=Cache, seed=1234):
    rng = np.random.default_rng(seed)
    keys = torch.from_numpy(rng.standard_normal((1, 1, 128, 512), dtype=np.float32) * 0.1).to(torch.float16).to(device)
    cache = cls(Ring(keys, offset, idx))
    cache.compressor_state["pooled"] = torch.from_numpy(
        rng.standard_normal((1, rows, 512), dtype=np.float32) * 0.1).to(torch.float16).to(device)
    cache.indexer_state["pooled"] = torch.from_numpy(
        rng.standard_normal((1, rows, 128), dtype=np.float32)).to(torch.float16).to(device)
    return cache
