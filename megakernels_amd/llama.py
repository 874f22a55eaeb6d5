"""Llama weights, rotary tables and KV cache in the layout the instruction VM
reads, plus a plain PyTorch forward used for prompt prefill.

What the decode path needs from reference ``megakernels/llama.py``:

* RMSNorm semantics (``llama.py:29-47``)
* interleaved rotary embedding helpers (``llama.py:136-174``) and the weight /
  table permutation that makes rotary pairs adjacent (``llama.py:453-475``)
* the embedding lookup (``llama.py:406-417``)
* rotary tables ``rope_cos/rope_sin [max_position, head_dim] fp32``
  (``llama.py:440-451``); the reference takes them from ``transformers``'
  ``LlamaRotaryEmbedding``, here the published llama3 frequency scaling is
  evaluated directly so the hot path does not depend on that package
* the KV cache ``[layers, batch, max_len, kv_heads, head_dim]`` (``llama.py:552-574``)
* weights stacked over layers (``llama.py:713-777``): ``qkv_proj`` is
  ``cat(q, k, v)`` along the output dimension.

The model is a plain container of tensors (no ``nn.Module``): the decode path
never runs autograd and the megakernel borrows raw device pointers.  The
attribute paths the generators use (``model.model.embed_tokens``,
``model.lm_head.input_norm.weight``, ``model.lm_head.lm_head.weight``,
``model.stacked_params``, ``model.stacked_kv_cache``) match the reference.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F
from torch import Tensor

from megakernels_amd.model_types import BatchState, DeviceType, ExtraModelConfig


# --------------------------------------------------------------------------
# configuration
# --------------------------------------------------------------------------


@dataclass
class LlamaConfig:
    """Architecture description with the attribute names of the Hugging Face
    ``LlamaConfig`` the reference passes around."""

    hidden_size: int = 2048
    intermediate_size: int = 8192
    num_hidden_layers: int = 16
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 64
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = field(
        default_factory=lambda: dict(
            rope_type="llama3",
            factor=32.0,
            low_freq_factor=1.0,
            high_freq_factor=4.0,
            original_max_position_embeddings=8192,
        )
    )
    max_position_embeddings: int = 131072
    tie_word_embeddings: bool = True

    @classmethod
    def llama_1b(cls) -> "LlamaConfig":
        """Llama-3.2-1B architecture."""
        return cls()

    @classmethod
    def llama_8b(cls) -> "LlamaConfig":
        """Llama-3.1-8B architecture."""
        cfg = cls(
            hidden_size=4096,
            intermediate_size=14336,
            num_hidden_layers=32,
            num_attention_heads=32,
            num_key_value_heads=8,
            head_dim=128,
            tie_word_embeddings=False,
        )
        cfg.rope_scaling["factor"] = 8.0
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "LlamaConfig":
        """Read a Hugging Face ``config.json``."""
        import json

        raw = json.loads(Path(path).read_text())
        known = {k: raw[k] for k in cls.__dataclass_fields__ if k in raw}
        if known.get("head_dim") is None:
            known["head_dim"] = raw["hidden_size"] // raw["num_attention_heads"]
        # transformers 4.x writes `rope_theta` and `rope_scaling`; 5.x writes one `rope_parameters`
        # dict holding the base as well.  A checkpoint without scaling has none: say so explicitly,
        # the dataclass default is the Llama-3.2 scaling.
        params = raw.get("rope_parameters")
        if params:
            params = dict(params)
            if "rope_theta" in params:
                known["rope_theta"] = float(params.pop("rope_theta"))
            known["rope_scaling"] = params
        elif "rope_scaling" not in raw:
            known["rope_scaling"] = None
        return cls(**known)


# --------------------------------------------------------------------------
# rotary tables
# --------------------------------------------------------------------------


def rope_inverse_frequencies(config: LlamaConfig) -> Tensor:
    """``inv_freq[i] = theta^(-2i/D)`` with the llama3 long-context scaling:
    wavelengths longer than ``orig/low_freq_factor`` are divided by ``factor``,
    wavelengths shorter than ``orig/high_freq_factor`` are kept, and the band
    in between is interpolated linearly in ``orig/wavelength``."""
    dim = config.head_dim
    exponents = torch.arange(0, dim, 2, dtype=torch.int64).float() / dim
    inv_freq = 1.0 / (config.rope_theta**exponents)
    scaling = config.rope_scaling
    if not scaling or scaling.get("rope_type", scaling.get("type")) in (None, "default"):
        return inv_freq
    if scaling.get("rope_type", scaling.get("type")) != "llama3":
        raise ValueError(f"unsupported rope scaling {scaling}")
    factor = scaling["factor"]
    low = scaling["low_freq_factor"]
    high = scaling["high_freq_factor"]
    orig = scaling["original_max_position_embeddings"]
    low_wavelen = orig / low
    high_wavelen = orig / high
    wavelen = 2 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_wavelen, inv_freq / factor, inv_freq)
    smooth = (orig / wavelen - low) / (high - low)
    blended = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
    return torch.where(medium, blended, scaled)


def rope_tables(config: LlamaConfig, num_positions: int | None = None):
    """``cos, sin`` of shape ``[positions, head_dim]`` in fp32, half-split
    layout (column ``i`` and ``i + D/2`` share a frequency)."""
    n = num_positions or config.max_position_embeddings
    inv_freq = rope_inverse_frequencies(config).float()
    angles = torch.arange(n, dtype=torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((angles, angles), dim=-1)
    return emb.cos(), emb.sin()


def interleave_permutation(head_dim: int, num_heads: int = 1) -> Tensor:
    """Row order ``[0, D/2, 1, D/2+1, ...]`` per head: puts the two members of
    each rotary pair next to each other (reference ``llama.py:453-461``)."""
    half = head_dim // 2
    one_head = torch.stack((torch.arange(half), torch.arange(half) + half), dim=-1).reshape(-1)
    return (one_head[None, :] + head_dim * torch.arange(num_heads)[:, None]).reshape(-1)


def rotate_half_interleaved(x: Tensor) -> Tensor:
    """``(x0, x1, x2, x3, ...) -> (-x1, x0, -x3, x2, ...)``."""
    pairs = x.reshape(*x.shape[:-1], -1, 2)
    return torch.stack((-pairs[..., 1], pairs[..., 0]), dim=-1).reshape(x.shape)


def apply_rotary_pos_emb_interleaved(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
    """Rotary embedding on adjacent pairs (reference ``llama.py:148-174``)."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (
        q * cos + rotate_half_interleaved(q) * sin,
        k * cos + rotate_half_interleaved(k) * sin,
    )


def rotate_half(x: Tensor) -> Tensor:
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
    """Half-split rotary embedding (the Hugging Face convention)."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """Llama RMSNorm: statistics in fp32, normalised value cast back to the
    input dtype, then multiplied by the weight (reference ``llama.py:38-47``)."""
    dtype = x.dtype
    x32 = x.float()
    x32 = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
    return weight * x32.to(dtype)


# --------------------------------------------------------------------------
# model container
# --------------------------------------------------------------------------


class _WeightHolder:
    """Object with a ``weight`` tensor, standing in for an ``nn.Linear`` /
    norm module wherever the generators only read ``.weight``."""

    def __init__(self, weight: Tensor):
        self.weight = weight


class LlamaEmbeddings(_WeightHolder):
    def __call__(self, batch_state: BatchState) -> BatchState:
        batch_state.hidden_states = F.embedding(batch_state.input_ids, self.weight)
        return batch_state

    # reference attribute path: model.model.embed_tokens.embed_tokens.weight
    @property
    def embed_tokens(self):
        return self


@dataclass
class StackedParams:
    qkv_proj: Tensor  # [L, (H + 2 KVH) D, hidden]
    o_proj: Tensor  # [L, hidden, H D]
    attn_ln_weight: Tensor  # [L, hidden]
    mlp_ln_weight: Tensor  # [L, hidden]
    up_proj: Tensor  # [L, inter, hidden]
    gate_proj: Tensor  # [L, inter, hidden]
    down_proj: Tensor  # [L, hidden, inter]


class LlamaModel:
    """Embedding table and rotary tables (``model.model`` in the reference)."""

    def __init__(self, config: LlamaConfig, embed_weight: Tensor, rope_cos: Tensor, rope_sin: Tensor):
        self.config = config
        self.embed_tokens = LlamaEmbeddings(embed_weight)
        self.rope_cos = rope_cos
        self.rope_sin = rope_sin


class LlamaLMHead:
    def __init__(self, config: LlamaConfig, norm_weight: Tensor, head_weight: Tensor):
        self.config = config
        self.input_norm = _WeightHolder(norm_weight)
        self.lm_head = _WeightHolder(head_weight)

    def __call__(self, batch_state: BatchState) -> BatchState:
        hidden = rms_norm(batch_state.hidden_states, self.input_norm.weight, self.config.rms_norm_eps)
        logits = F.linear(hidden, self.lm_head.weight)
        batch_state.output_ids = logits.argmax(dim=-1)
        return batch_state


class LlamaForCausalLM:
    def __init__(
        self,
        config: LlamaConfig,
        extra_config: ExtraModelConfig,
        stacked_params: StackedParams,
        embed_weight: Tensor,
        final_norm_weight: Tensor,
        lm_head_weight: Tensor,
        rope_cos: Tensor,
        rope_sin: Tensor,
    ):
        self.config = config
        self.extra_config = extra_config
        self.stacked_params = stacked_params
        self.model = LlamaModel(config, embed_weight, rope_cos, rope_sin)
        self.lm_head = LlamaLMHead(config, final_norm_weight, lm_head_weight)
        self.device = embed_weight.device
        self.dtype = embed_weight.dtype
        self.stacked_kv_cache: tuple[Tensor, Tensor] | None = None

    # ---- construction ----------------------------------------------------

    @classmethod
    def from_random(
        cls,
        config: LlamaConfig,
        extra_config: ExtraModelConfig | None = None,
        seed: int = 0,
        device: DeviceType = "cpu",
        dtype: torch.dtype = torch.bfloat16,
        std: float = 0.02,
        draw_device: DeviceType | None = None,
    ) -> "LlamaForCausalLM":
        """Random-initialised model: every matrix is drawn ``N(0, std)`` in fp32
        from a CPU generator seeded with ``seed`` and cast to ``dtype``; norm
        weights are one.  Draw order: embedding; per layer q, k, v, o, up, gate,
        down; then the LM head when it is not tied to the embedding.  The same
        seed yields the same bits on every host, so a CPU checker and the GPU
        run can be fed identical weights.  ``draw_device``: draw with that
        device's generator instead (a GPU fills the 8B architecture in seconds
        where the CPU generator takes minutes; the bits then belong to that
        generator, and a CPU twin is made with ``.to("cpu")``)."""
        extra_config = extra_config or ExtraModelConfig(interleave_rope=True)
        draw_device = torch.device(draw_device or "cpu")
        gen = torch.Generator(device=draw_device).manual_seed(seed)
        c = config
        H, KVH, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        L, hid, inter = c.num_hidden_layers, c.hidden_size, c.intermediate_size

        def draw(rows, cols):
            return torch.empty(rows, cols, dtype=torch.float32, device=draw_device).normal_(0.0, std, generator=gen).to(dtype)

        def stack(*shape):
            return torch.empty(*shape, dtype=dtype, device=draw_device)

        embed = draw(c.vocab_size, hid)
        qkv = stack(L, (H + 2 * KVH) * D, hid)
        o = stack(L, hid, H * D)
        up = stack(L, inter, hid)
        gate = stack(L, inter, hid)
        down = stack(L, hid, inter)
        q_perm = interleave_permutation(D, H).to(draw_device)
        k_perm = interleave_permutation(D, KVH).to(draw_device)
        for layer in range(L):
            q, k, v = draw(H * D, hid), draw(KVH * D, hid), draw(KVH * D, hid)
            if extra_config.interleave_rope:
                q, k = q[q_perm], k[k_perm]
            qkv[layer] = torch.cat((q, k, v), dim=0)
            o[layer] = draw(hid, H * D)
            up[layer] = draw(inter, hid)
            gate[layer] = draw(inter, hid)
            down[layer] = draw(hid, inter)
        head = embed if c.tie_word_embeddings else draw(c.vocab_size, hid)
        stacked = StackedParams(
            qkv_proj=qkv,
            o_proj=o,
            attn_ln_weight=torch.ones(L, hid, dtype=dtype),
            mlp_ln_weight=torch.ones(L, hid, dtype=dtype),
            up_proj=up,
            gate_proj=gate,
            down_proj=down,
        )
        return cls._assemble(
            c, extra_config, stacked, embed, torch.ones(hid, dtype=dtype), head, device
        )

    @classmethod
    def from_pretrained(
        cls,
        model_path: str | Path,
        extra_config: ExtraModelConfig | None = None,
        device: DeviceType = "cpu",
        dtype: torch.dtype = torch.bfloat16,
    ) -> "LlamaForCausalLM":
        """Load a local Hugging Face checkpoint directory (``config.json`` and
        ``*.safetensors``) into the stacked layout, applying the rotary-pair
        permutation to the q/k rows when ``interleave_rope`` is set
        (reference ``llama.py:583-638,640-663``).  Nothing is downloaded."""
        from safetensors import safe_open

        extra_config = extra_config or ExtraModelConfig(interleave_rope=True)
        path = Path(model_path)
        if not path.is_dir():
            raise FileNotFoundError(
                f"{path} is not a local checkpoint directory; this build does not download models"
            )
        c = LlamaConfig.from_json(path / "config.json")
        if extra_config.rope_scaling is not None:
            c.rope_scaling = extra_config.rope_scaling
        tensors: dict[str, Tensor] = {}
        files = sorted(path.glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no *.safetensors under {path}")
        for file in files:
            with safe_open(file, framework="pt", device="cpu") as f:
                for key in f.keys():
                    tensors[key] = f.get_tensor(key).to(dtype)
        H, KVH, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        q_perm = interleave_permutation(D, H)
        k_perm = interleave_permutation(D, KVH)

        def layer_tensor(layer, name):
            return tensors[f"model.layers.{layer}.{name}.weight"]

        qkv, o, up, gate, down, ln1, ln2 = [], [], [], [], [], [], []
        for layer in range(c.num_hidden_layers):
            q = layer_tensor(layer, "self_attn.q_proj")
            k = layer_tensor(layer, "self_attn.k_proj")
            v = layer_tensor(layer, "self_attn.v_proj")
            if extra_config.interleave_rope:
                q, k = q[q_perm], k[k_perm]
            qkv.append(torch.cat((q, k, v), dim=0))
            o.append(layer_tensor(layer, "self_attn.o_proj"))
            up.append(layer_tensor(layer, "mlp.up_proj"))
            gate.append(layer_tensor(layer, "mlp.gate_proj"))
            down.append(layer_tensor(layer, "mlp.down_proj"))
            ln1.append(layer_tensor(layer, "input_layernorm"))
            ln2.append(layer_tensor(layer, "post_attention_layernorm"))
        stacked = StackedParams(
            qkv_proj=torch.stack(qkv),
            o_proj=torch.stack(o),
            attn_ln_weight=torch.stack(ln1),
            mlp_ln_weight=torch.stack(ln2),
            up_proj=torch.stack(up),
            gate_proj=torch.stack(gate),
            down_proj=torch.stack(down),
        )
        embed = tensors["model.embed_tokens.weight"]
        head = embed if c.tie_word_embeddings else tensors["lm_head.weight"]
        return cls._assemble(c, extra_config, stacked, embed, tensors["model.norm.weight"], head, device)

    @classmethod
    def _assemble(cls, config, extra_config, stacked, embed, final_norm, head, device):
        cos, sin = rope_tables(config)
        if extra_config.interleave_rope:
            cols = interleave_permutation(config.head_dim)
            cos, sin = cos[:, cols].contiguous(), sin[:, cols].contiguous()
        tied = head is embed

        def move(t):
            return t.to(device).contiguous()

        stacked = StackedParams(**{k: move(v) for k, v in vars(stacked).items()})
        embed = move(embed)
        head = embed if tied else move(head)
        model = cls(config, extra_config, stacked, embed, move(final_norm), head, move(cos), move(sin))
        model.setup_caches()
        return model

    def to(self, device: DeviceType) -> "LlamaForCausalLM":
        """A copy of the model (weights, rope tables, fresh zeroed KV cache) on
        ``device``; a tied LM head stays tied."""
        emb = self.model.embed_tokens.weight
        head = self.lm_head.lm_head.weight
        return type(self)._assemble_moved(self, torch.device(device), head is emb)

    @classmethod
    def _assemble_moved(cls, src: "LlamaForCausalLM", device, tied: bool):
        def move(t):
            return t.to(device).contiguous()

        stacked = StackedParams(**{k: move(v) for k, v in vars(src.stacked_params).items()})
        embed = move(src.model.embed_tokens.weight)
        head = embed if tied else move(src.lm_head.lm_head.weight)
        model = cls(
            src.config, src.extra_config, stacked, embed, move(src.lm_head.input_norm.weight), head,
            move(src.model.rope_cos), move(src.model.rope_sin),
        )
        model.setup_caches()
        return model

    def setup_caches(self):
        """Zeroed K and V caches ``[L, batch, max_len, KVH, D]``
        (reference ``llama.py:552-567``)."""
        c = self.config
        shape = (
            c.num_hidden_layers,
            self.extra_config.max_batch_size,
            self.extra_config.max_len_override or c.max_position_embeddings,
            c.num_key_value_heads,
            c.head_dim,
        )
        k_cache = torch.zeros(shape, device=self.device, dtype=self.dtype)
        self.stacked_kv_cache = (k_cache, torch.zeros_like(k_cache))

    # ---- plain forward (prefill and the torch generator) ------------------

    @torch.inference_mode()
    def forward(self, batch_state: BatchState) -> BatchState:
        """Dense forward over ``input_ids [B, S]`` at ``position_ids [S]``;
        writes the KV cache at those positions and returns greedy
        ``output_ids [B, S]`` (reference ``llama.py:232-296,328-348,384-403``).
        ``S > 1`` is a prefill from position 0 with a causal mask, ``S == 1``
        a decode step attending to ``seq_len`` cached positions."""
        c = self.config
        p = self.stacked_params
        ids = batch_state.input_ids
        if ids.ndim == 1:
            ids = ids[None]
        pos = batch_state.position_ids
        if pos.ndim == 2:
            pos = pos[0]
        B, S = ids.shape
        H, KVH, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        cos, sin = self.model.rope_cos[pos], self.model.rope_sin[pos]
        rope = apply_rotary_pos_emb_interleaved if self.extra_config.interleave_rope else apply_rotary_pos_emb
        k_cache, v_cache = self.stacked_kv_cache
        seq_len = batch_state.seq_len if S == 1 else S

        h = F.embedding(ids, self.model.embed_tokens.weight)
        for layer in range(c.num_hidden_layers):
            x = rms_norm(h, p.attn_ln_weight[layer], c.rms_norm_eps)
            qkv = F.linear(x, p.qkv_proj[layer])
            q, k, v = qkv.split([H * D, KVH * D, KVH * D], dim=-1)
            q = q.view(B, S, H, D)
            k = k.view(B, S, KVH, D)
            v = v.view(B, S, KVH, D)
            q, k = rope(q, k, cos, sin, unsqueeze_dim=-2)
            q, k = q.to(h.dtype), k.to(h.dtype)
            k_cache[layer][:B, pos] = k
            v_cache[layer][:B, pos] = v
            if S > 1:
                keys, values, causal = k, v, True
            else:
                keys, values, causal = k_cache[layer][:B, :seq_len], v_cache[layer][:B, :seq_len], False
            attn = F.scaled_dot_product_attention(
                q.transpose(1, 2),
                keys.transpose(1, 2),
                values.transpose(1, 2),
                is_causal=causal,
                enable_gqa=True,
            )
            attn = attn.transpose(1, 2).reshape(B, S, H * D)
            h = h + F.linear(attn, p.o_proj[layer])
            x = rms_norm(h, p.mlp_ln_weight[layer], c.rms_norm_eps)
            prod = F.silu(F.linear(x, p.gate_proj[layer])) * F.linear(x, p.up_proj[layer])
            h = h + F.linear(prod, p.down_proj[layer])
        out = BatchState(input_ids=ids, position_ids=pos, seq_len=seq_len, hidden_states=h)
        return self.lm_head(out)

    __call__ = forward
