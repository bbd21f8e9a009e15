"""A hybrid GatedDeltaNet / attention / mixture-of-experts model served two ways over ONE set of ops.

``TrainerModel`` scores whole packed sequences in one pass (the role of the reference's Megatron
trainer forward); ``RolloutEngine`` prefills prompts and then decodes token by token out of state
pools and a key/value cache (the role of its vLLM rollout forward, isoexec/runtimes/vllm/
gptmodel_vllm.py). Both are thin drivers over ``_Blocks``, which holds every projection, norm and
mixture call, so the two runtimes differ only in how tokens are cut into calls and where sequence
state lives -- the things the kernels are invariant to. The logprob a rollout records for a sampled
token therefore equals, bit for bit, the logprob the trainer later assigns to it.

Layer layout (pre-norm residual stream, hidden H):
    h -> norm -> mixer -> (+h, norm) -> mixture of experts -> (+h) -> next layer
    mixer = GatedDeltaNet (in_proj -> causal conv -> l2norm/gate -> delta-rule scan -> gated norm ->
            out_proj) on three layers of four, causal grouped-query attention with rotary embedding
            (qkv_proj -> rope -> attention -> o_proj) on the fourth.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..debug.trace import get_tracer
from ..ops.attention.varlen_attn import KVCache, varlen_attention
from ..ops.gdn.gdn_ops import conv_packed, gdn_native_core, gdn_native_core_normed
from ..ops.gdn.gdn_cpr import gdn_native_cpr_fwd
from ..ops.gdn.gdn_cpr_state import CprGDN
from ..ops.gdn.gdn_recurrent_state import RecurrentGDN
from ..ops.logprobs.rowinv import leaves, sampled_forward
from ..ops.mm.mm_hip import linear_nt, pack_nt_decode
from ..ops.moe.moe_hip import moe_ffn_forward
from ..ops.norms.fused_outnorm import fused_add_rms_norm_gamma, fused_gated_out_norm, fused_rms_norm_gamma
from ..ops.rope.rope_hip import apply_rope_, rope_tables


@dataclass(frozen=True)
class HybridConfig:
    hidden: int = 2048
    vocab: int = 151936
    layers: int = 8
    attention_every: int = 4  # layers 3, 7, ... (0-based) are attention; the rest GatedDeltaNet
    # GatedDeltaNet
    gdn_k_heads: int = 16
    gdn_v_heads: int = 32
    gdn_head_dim: int = 128
    conv_width: int = 4
    # delta-rule kernel of every site: "recurrent", or "cpr" (fp32 chain at chunk boundaries, running state
    # re-snapshotted in the wire dtype every gdn_chunk tokens); trainer and engine must run the same one
    gdn_kernel: str = "recurrent"
    gdn_chunk: int = 64
    # attention
    q_heads: int = 32
    kv_heads: int = 4
    head_dim: int = 128
    rope_theta: float = 1.0e6
    max_positions: int = 4096
    # mixture of experts
    experts: int = 128
    topk: int = 8
    expert_inter: int = 768
    # what a token's k expert rows are summed in by the combine: "fp32" (the contract's default) or "bf16"
    moe_combine_dtype: str = "fp32"
    eps: float = 1.0e-6

    def is_attention(self, layer: int) -> bool:
        return (layer + 1) % self.attention_every == 0

    def profile(self):
        """The model declaration of THIS configuration: the production declaration with the widths and kernel
        choices that reach the contract replaced by this configuration's."""
        from ..models import qwen3_5
        from ..models.profile import RouterProfile

        return qwen3_5.PROFILE.with_overrides(
            model=f"hybrid-{self.layers}l-{self.experts}e", name_patterns=(),
            router=RouterProfile(topk=self.topk, num_experts=self.experts),
            gdn_kernel=self.gdn_kernel, gdn_chunk_size=self.gdn_chunk, moe_combine_dtype=self.moe_combine_dtype)

    @property
    def gdn_qkv(self) -> int:
        return 2 * self.gdn_k_heads * self.gdn_head_dim + self.gdn_v_heads * self.gdn_head_dim

    @property
    def gdn_z(self) -> int:
        return self.gdn_v_heads * self.gdn_head_dim


def _normal(shape, std, gen, device, dtype=torch.bfloat16):
    """N(0, std) drawn from ``gen``. A generator that lives on the host draws on the host (in pieces of at most 64 M
    values, so the fp32 staging stays small) and the pieces are cast on the device: the values then do not depend on
    which GPU, or which vendor's GPU, runs the model."""
    if gen.device.type == torch.device(device).type:
        return (torch.randn(shape, generator=gen, device=device) * std).to(dtype)
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    step = 1 << 26
    for lo in range(0, flat.numel(), step):
        n = min(step, flat.numel() - lo)
        flat[lo : lo + n] = (torch.randn(n, generator=gen).to(device, non_blocking=False) * std).to(dtype)
    return out


@dataclass
class HybridWeights:
    """Random-initialised parameters (N(0, 0.02) projections, zero-centred norm gains)."""

    embed: torch.Tensor
    lm_head: torch.Tensor
    final_norm: torch.Tensor
    layers: list = field(default_factory=list)

    @classmethod
    def make(cls, cfg: HybridConfig, seed: int = 0, device="cuda", host_rng: bool = False) -> "HybridWeights":
        g = torch.Generator(device="cpu" if host_rng else device)
        g.manual_seed(seed)
        H = cfg.hidden
        w = cls(embed=_normal((cfg.vocab, H), 1.0, g, device), lm_head=_normal((cfg.vocab, H), 0.02, g, device),
                final_norm=_normal((H,), 0.02, g, device))
        for i in range(cfg.layers):
            lw = {
                "pre_norm": _normal((H,), 0.02, g, device),
                "post_norm": _normal((H,), 0.02, g, device),
                "router": _normal((cfg.experts, H), 0.02, g, device),
                "w1": _normal((cfg.experts, 2 * cfg.expert_inter, H), 0.02, g, device),
                "w2": _normal((cfg.experts, H, cfg.expert_inter), 0.02, g, device),
            }
            if cfg.is_attention(i):
                lw["qkv_proj"] = _normal(((cfg.q_heads + 2 * cfg.kv_heads) * cfg.head_dim, H), 0.02, g, device)
                lw["o_proj"] = _normal((H, cfg.q_heads * cfg.head_dim), 0.02, g, device)
            else:
                lw["in_proj"] = _normal((cfg.gdn_qkv + cfg.gdn_z + 2 * cfg.gdn_v_heads, H), 0.02, g, device)
                lw["conv_weight"] = _normal((cfg.gdn_qkv, cfg.conv_width), 0.4, g, device)
                lw["conv_bias"] = _normal((cfg.gdn_qkv,), 0.1, g, device)
                lw["A_log"] = _normal((cfg.gdn_v_heads,), 0.3, g, device, torch.float32)
                lw["dt_bias"] = _normal((cfg.gdn_v_heads,), 0.3, g, device, torch.float32)
                lw["out_norm"] = _normal((cfg.gdn_head_dim,), 0.02, g, device)
                lw["out_proj"] = _normal((H, cfg.gdn_z), 0.02, g, device)
            w.layers.append(lw)
        return w


def check_lengths(cfg: "HybridConfig", lens, what: str) -> None:
    """Every sequence must fit the rotary tables (``cfg.max_positions`` rows): positions are 0 .. len-1."""
    longest = int(max(lens)) if len(lens) else 0
    if longest > cfg.max_positions:
        raise ValueError(f"[isoexec-amd] {what}: a sequence of {longest} tokens exceeds max_positions = "
                         f"{cfg.max_positions} (the rotary tables hold that many positions)")


def _linear(x, w):
    out = linear_nt(x, w)
    if out is None:
        raise RuntimeError(f"[isoexec-amd] GEMM declined for x {tuple(x.shape)} {x.dtype} w {tuple(w.shape)}")
    return out


class _Blocks:
    """Every weight-bearing call of a layer, shared by both runtimes."""

    def __init__(self, cfg: HybridConfig, weights: HybridWeights):
        self.cfg, self.w = cfg, weights
        dev = weights.embed.device
        self.cos, self.sin = rope_tables(cfg.max_positions, cfg.head_dim, cfg.rope_theta, device=dev)
        # a debug.regions.RegionLog or the process's debug.trace.Tracer (there is one when SKYRL_ISOEXEC_DEBUG_TRACE names
        # a directory), else None: when set, the residual stream's per-layer outputs are digested on the device as they
        # are produced, so that two runtimes' passes over the same tokens can be compared region by region
        self.region_log = get_tracer()
        # a list, or None: when set, every mixture call appends its top-k expert ids [T, k] (layer order)
        self.routing_log = None
        # layer -> fragment-packed copies of the experts' matrices (pack_expert_weights): read by decode-size batches only
        self.packed_experts = {}
        # (layer, name) or "lm_head" -> mm_hip.PackedWeight of a wide dense weight (pack_dense_weights): products of
        # at most 64 rows stream the packed copy, every other product reads the weight itself
        self.packed_dense = {}

    def pack_expert_weights(self) -> int:
        """Make the packed copies of the experts' matrices that decode-size batches stream (one pass over each matrix; a
        second copy of them in memory). To be called again after a weight sync. Returns the bytes they take."""
        from ..ops.moe.moe_hip import pack_decode

        total = 0
        for i, lw in enumerate(self.w.layers):
            packed = pack_decode(lw["w1"], lw["w2"])
            if packed is not None:
                self.packed_experts[i] = packed
                total += sum(t.numel() * t.element_size() for t in packed)
        return total

    # dense weights with at least this many rows have enough 32-row units for the streaming form to beat the ring tiles
    # at 64 rows (12352 rows: 15.9 against 17.9 us; 5120 rows: 12.2 against 10.8)
    PACK_DENSE_MIN_ROWS = 12288

    def pack_dense_weights(self) -> int:
        """Make the packed copies of the wide dense weights (the GDN input projection, the LM head) that products of at
        most 64 rows stream. To be called again after a weight sync. Returns the bytes they take."""
        total = 0
        todo = [((i, "in_proj"), lw["in_proj"]) for i, lw in enumerate(self.w.layers) if "in_proj" in lw]
        todo.append(("lm_head", self.w.lm_head))
        for key, weight in todo:
            if weight.shape[0] < self.PACK_DENSE_MIN_ROWS:
                continue
            packed = pack_nt_decode(weight)
            if packed is not None:
                self.packed_dense[key] = packed
                total += packed.packed.numel() * packed.packed.element_size()
        return total

    def _dense(self, key, weight):
        return self.packed_dense.get(key, weight)

    def _note(self, region: str, layer, out) -> None:
        if self.region_log is not None:
            self.region_log.record(region, out, layer=layer)

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        return self.w.embed.index_select(0, tokens)

    def gdn_in(self, layer: int, x: torch.Tensor):
        """-> views of one projection buffer: pre-conv ``qkv [T, D]``, ``z [T, HV, V]``, ``b``, ``a [T, HV]``."""
        c = self.cfg
        proj = _linear(x, self._dense((layer, "in_proj"), self.w.layers[layer]["in_proj"]))
        qkv = proj[:, : c.gdn_qkv]
        z = proj[:, c.gdn_qkv : c.gdn_qkv + c.gdn_z].unflatten(1, (c.gdn_v_heads, c.gdn_head_dim))
        b = proj[:, c.gdn_qkv + c.gdn_z : c.gdn_qkv + c.gdn_z + c.gdn_v_heads]
        a = proj[:, c.gdn_qkv + c.gdn_z + c.gdn_v_heads :]
        return qkv, z, b, a

    @property
    def fuse_ops(self) -> bool:
        """Whether the runtimes may fold neighbouring ops into one launch (conv + l2norm, scan + gated output norm,
        combine + add + norm). Not while a region log or the trace is attached: each op's output is then a region of its
        own, and both sides have to cut the computation at the same points. Same bits either way."""
        return self.region_log is None

    def gdn_out(self, layer: int, o: torch.Tensor, z: torch.Tensor, normed: bool = False) -> torch.Tensor:
        """Gated output norm (unless the scan applied it already: ``normed``) and the output projection."""
        lw = self.w.layers[layer]
        y = o if normed else fused_gated_out_norm(o, z, lw["out_norm"], self.cfg.eps)
        return _linear(y.reshape(o.shape[0], -1), lw["out_proj"])

    def gdn_gated_norm(self, layer: int, z: torch.Tensor) -> tuple:
        """What a scan needs to apply the layer's gated output norm itself: ``(gate, weight, eps, zero_centered)``."""
        return z, self.w.layers[layer]["out_norm"], self.cfg.eps, True

    def attn_qkv(self, layer: int, x: torch.Tensor, positions: torch.Tensor):
        """-> views ``q [T, HQ, D]``, ``k, v [T, HKV, D]`` of one projection buffer, q and k rotated."""
        c = self.cfg
        proj = _linear(x, self.w.layers[layer]["qkv_proj"])
        nq, nk = c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        q = proj[:, :nq].unflatten(1, (c.q_heads, c.head_dim))
        k = proj[:, nq : nq + nk].unflatten(1, (c.kv_heads, c.head_dim))
        v = proj[:, nq + nk :].unflatten(1, (c.kv_heads, c.head_dim))
        # q and k are adjacent column blocks with one head size: one launch rotates the q and kv heads of a token
        apply_rope_(proj[:, : nq + nk].unflatten(1, (c.q_heads + c.kv_heads, c.head_dim)), self.cos, self.sin, positions)
        return q, k, v

    def attn_out(self, layer: int, o: torch.Tensor) -> torch.Tensor:
        return _linear(o.view(o.shape[0], -1), self.w.layers[layer]["o_proj"])

    def moe(self, layer: int, x: torch.Tensor, add_norm=None):
        """The layer's mixture of experts; with ``add_norm = (residual, weight, eps)`` also the residual add and the next
        norm, folded into the combine's launch: returns ``(normed, h)`` then."""
        lw = self.w.layers[layer]
        return moe_ffn_forward(x, lw["router"], lw["w1"], lw["w2"], self.cfg.topk, pre_softmax=True,
                               fp32_combine=self.cfg.moe_combine_dtype == "fp32", routing_out=self.routing_log,
                               add_norm=add_norm, packed=self.packed_experts.get(layer))

    def run_layers(self, h: torch.Tensor, mixer) -> torch.Tensor:
        """The residual stream over all layers; ``mixer(layer, x)`` is the runtime's own part."""
        c = self.cfg
        x = fused_rms_norm_gamma(h, self.w.layers[0]["pre_norm"], c.eps)
        for i in range(c.layers):
            lw = self.w.layers[i]
            mixed = mixer(i, x)
            self._note("attention.varlen" if c.is_attention(i) else "gdn.core", i, mixed)
            x, h = fused_add_rms_norm_gamma(mixed, h, lw["post_norm"], c.eps)
            nxt = self.w.layers[i + 1]["pre_norm"] if i + 1 < c.layers else self.w.final_norm
            if self.fuse_ops:
                x, h = self.moe(i, x, add_norm=(h, nxt, c.eps))
            else:  # the mixture's own output is a region of the comparison: keep it as a tensor
                delta = self.moe(i, x)
                self._note("moe.combine", i, delta)
                x, h = fused_add_rms_norm_gamma(delta, h, nxt, c.eps)
            self._note("norms.rms", i, (x, h))
        return x  # final-normed hidden states

    def logits(self, x: torch.Tensor, want_row_max: bool = False):
        got = linear_nt(x, self._dense("lm_head", self.w.lm_head), want_row_max=want_row_max)
        if got is None:
            raise RuntimeError("[isoexec-amd] LM-head GEMM declined")
        return got

    def sampled_logprobs(self, x: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
        logits, row_max = self.logits(x, want_row_max=True)
        got = sampled_forward(logits, targets, leaves(), row_max=row_max)
        if got is None:
            raise RuntimeError(f"[isoexec-amd] the log-softmax kernel declined vocab {logits.shape[1]} with "
                               f"{leaves()} leaves (the vocabulary must divide into the leaves)")
        return got[0]


def bound_implementations(cfg: HybridConfig) -> dict:
    """op -> (impl id, the callable these runtimes bind for it, the constants it runs with). Written from what the
    code above calls, not read back from a contract, so that comparing it with a contract says something."""
    scan = gdn_native_cpr_fwd if cfg.gdn_kernel == "cpr" else gdn_native_core
    from ..ops.logprobs.rowinv import BLOCK

    return {
        "mm": ("hip_mfma_batch_invariant", linear_nt, None),
        "norms.rms": ("hip_fused", fused_add_rms_norm_gamma, None),
        "norms.gated_out": ("hip_fused", fused_gated_out_norm, None),
        "attention.varlen": ("hip_varlen_ns1", varlen_attention, {"num_splits": 1}),
        "rope.rope": ("hip_rope", apply_rope_, None),
        "gdn.conv": ("hip_causal_conv", conv_packed, None),
        "gdn.core": ("hip_fused_recurrent", scan, {"kernel": cfg.gdn_kernel}),
        "gdn.state": ("hip_private_pool", CprGDN if cfg.gdn_kernel == "cpr" else RecurrentGDN, {"ssm_cache_dtype": "float32"}),
        "moe.router": ("hip_fused_topk", moe_ffn_forward, {"topk": cfg.topk, "experts": cfg.experts, "score": "softmax_then_topk"}),
        "moe.dispatch": ("hip_bitmask_index", moe_ffn_forward, None),
        "moe.experts": ("hip_grouped_mfma", moe_ffn_forward, None),
        "moe.combine": ("hip_fixed_order", moe_ffn_forward, {"leaf_dtype": cfg.moe_combine_dtype}),
        "logprobs.log_softmax": ("hip_rowinv_leaftree", sampled_forward, {"leaves": leaves(), "block": BLOCK, "accum": "kahan_fp32"}),
        "logprobs.lm_head_slice": ("sampled_rows", _Blocks.sampled_logprobs, None),
    }


def record_runtime_installs(cfg: HybridConfig, side: str, registry=None) -> int:
    """File, for every op above, an install record at each site of ``side`` ("trainer" / "engine") the op exists at.
    Returns the number of (op, site) keys recorded."""
    from ..core import enforce, fingerprint
    from ..core.registry_build import build_registry

    registry = registry or build_registry()
    count = 0
    for op, (impl_id, fn, pins) in bound_implementations(cfg).items():
        sites = [site for site in registry.get_op(op).sites if site in enforce.SIDES[side]]
        fingerprint.record_installs(op, sites, impl_id, fn, pins)
        count += len(sites)
    return count


class TrainerModel:
    """Full-sequence scoring over packed sequences."""

    def __init__(self, cfg: HybridConfig, weights: HybridWeights):
        self.cfg, self.blocks = cfg, _Blocks(cfg, weights)

    @torch.no_grad()
    def hidden_states(self, tokens: torch.Tensor, lens: list) -> torch.Tensor:
        """``tokens`` int64 [sum(lens)] packed; returns the final-normed hidden states [sum(lens), H]."""
        b, c = self.blocks, self.cfg
        check_lengths(c, lens, "trainer pass")
        dev = tokens.device
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        cu = torch.from_numpy(offs).to(dev)
        positions = torch.from_numpy(np.concatenate([np.arange(n, dtype=np.int32) for n in lens])).to(dev)
        max_len = int(max(lens))

        def mixer(i, x):
            lw = b.w.layers[i]
            if c.is_attention(i):
                q, k, v = b.attn_qkv(i, x, positions)
                return b.attn_out(i, varlen_attention(q, k, v, cu, max_len))
            qkv, z, bb, a = b.gdn_in(i, x)
            kd = c.gdn_k_heads * c.gdn_head_dim
            # the recurrent form takes q and k normalised by the convolution's own launch and hands its output to the
            # gated norm inside the scan's (where the library serves those forms; the same bits as the ops apart)
            fused = b.fuse_ops and c.gdn_kernel != "cpr"
            y = conv_packed(qkv, lw["conv_weight"], lw["conv_bias"], cu_seqlens=cu, l2norm_qk=2 * kd if fused else 0,
                            head_k_dim=c.gdn_head_dim)
            q = y[:, :kd].unflatten(1, (c.gdn_k_heads, c.gdn_head_dim))
            k = y[:, kd : 2 * kd].unflatten(1, (c.gdn_k_heads, c.gdn_head_dim))
            v = y[:, 2 * kd :].unflatten(1, (c.gdn_v_heads, c.gdn_head_dim))
            if c.gdn_kernel == "cpr":
                o = gdn_native_cpr_fwd(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), a, bb, lw["A_log"], lw["dt_bias"],
                                       cu_seqlens=cu, chunk_size=c.gdn_chunk)
            elif fused:
                o = gdn_native_core_normed(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), a, bb, lw["A_log"],
                                           lw["dt_bias"], cu_seqlens=cu, gated_norm=b.gdn_gated_norm(i, z))
                return b.gdn_out(i, o[0], z, normed=True)
            else:
                o = gdn_native_core(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), a, bb, lw["A_log"], lw["dt_bias"], cu_seqlens=cu)
            return b.gdn_out(i, o[0], z)

        return b.run_layers(b.embed(tokens), mixer)

    @torch.no_grad()
    def response_logprobs(self, tokens: torch.Tensor, lens: list, prompt_lens: list) -> list:
        """Logprob of every response token: for sequence n, tokens ``prompt_lens[n] .. lens[n]-1``,
        each scored from the hidden state one position earlier. Returns a list of fp32 tensors."""
        x = self.hidden_states(tokens, lens)
        rows, targets, start = [], [], 0
        for n, p in zip(lens, prompt_lens):
            rows.append(torch.arange(start + p - 1, start + n - 1, device=tokens.device))
            targets.append(tokens[start + p : start + n])
            start += n
        lp = self.blocks.sampled_logprobs(x.index_select(0, torch.cat(rows)), torch.cat(targets))
        return list(lp.split([n - p for n, p in zip(lens, prompt_lens)]))


class RolloutEngine:
    """Prefill, then one token per step per sequence, out of per-layer state."""

    def __init__(self, cfg: HybridConfig, weights: HybridWeights, max_num_seqs: int, max_len: int,
                 pack_expert_weights: bool = True):
        if max_len > cfg.max_positions:
            raise ValueError(f"[isoexec-amd] engine max_len = {max_len} exceeds max_positions = {cfg.max_positions} "
                             "(the rotary tables hold that many positions)")
        self.cfg, self.blocks = cfg, _Blocks(cfg, weights)
        if pack_expert_weights:
            # the engine's decode steps stream every touched expert's weights, the input projections and the LM head:
            # from contiguous packed copies
            self.blocks.pack_expert_weights()
            self.blocks.pack_dense_weights()
        dev = weights.embed.device
        self.max_len = max_len
        self.gdn, self.kv = {}, {}
        for i in range(cfg.layers):
            lw = weights.layers[i]
            if cfg.is_attention(i):
                self.kv[i] = KVCache(max_num_seqs, max_len, cfg.kv_heads, cfg.head_dim, device=dev)
            else:
                kw = dict(capacity=max_num_seqs, conv_weight=lw["conv_weight"], conv_bias=lw["conv_bias"],
                          A_log=lw["A_log"], dt_bias=lw["dt_bias"], num_k_heads=cfg.gdn_k_heads,
                          head_k_dim=cfg.gdn_head_dim, num_v_heads=cfg.gdn_v_heads, head_v_dim=cfg.gdn_head_dim,
                          device=dev, driver_managed=True)
                self.gdn[i] = CprGDN(chunk_size=cfg.gdn_chunk, **kw) if cfg.gdn_kernel == "cpr" else RecurrentGDN(**kw)
        # One row table names a request's place in the key/value caches; the GatedDeltaNet layers keep
        # their own (identical) tables so each can be released or evicted with its pool.
        self.kv_rows: dict[int, int] = {}
        self.free_kv_rows = list(range(max_num_seqs, 0, -1))
        self.context: dict[int, int] = {}

    def _kv_row(self, slot: int) -> int:
        if slot not in self.kv_rows:
            if not self.free_kv_rows:
                raise RuntimeError("[isoexec-amd] key/value cache exhausted: release finished requests first")
            self.kv_rows[slot] = self.free_kv_rows.pop()
        return self.kv_rows[slot]

    def release(self, slot: int) -> None:
        for layer in self.gdn.values():
            layer.release_slot(slot)
        row = self.kv_rows.pop(slot, None)
        if row is not None:
            self.free_kv_rows.append(row)
        self.context.pop(slot, None)

    @torch.no_grad()
    def prefill(self, slots: list, tokens: torch.Tensor, lens: list) -> torch.Tensor:
        """Prompts packed in ``tokens``; returns the final-normed hidden state of each prompt's LAST
        token ``[N, H]`` (the row the first response token is sampled from)."""
        b, c = self.blocks, self.cfg
        check_lengths(c, lens, "prefill")
        if int(max(lens)) > self.max_len:
            raise ValueError(f"[isoexec-amd] prefill: a prompt of {int(max(lens))} tokens exceeds the cache length {self.max_len}")
        dev = tokens.device
        offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        cu = torch.from_numpy(offs).to(dev)
        positions = torch.from_numpy(np.concatenate([np.arange(n, dtype=np.int32) for n in lens])).to(dev)
        rows = [self._kv_row(s) for s in slots]
        kv_index = torch.from_numpy(np.concatenate([r * self.max_len + np.arange(n, dtype=np.int64) for r, n in zip(rows, lens)])).to(dev)
        kv_start = torch.tensor([r * self.max_len for r in rows], dtype=torch.int64, device=dev)
        slots_t = torch.tensor(slots, dtype=torch.int64, device=dev)
        max_len = int(max(lens))
        qsl = [int(o) for o in offs]

        def mixer(i, x):
            if c.is_attention(i):
                q, k, v = b.attn_qkv(i, x, positions)
                self.kv[i].write(kv_index, k, v)
                kf, vf = self.kv[i].flat()
                return b.attn_out(i, varlen_attention(q, kf, vf, cu, max_len, kv_start=kv_start))
            qkv, z, bb, a = b.gdn_in(i, x)
            layer = self.gdn[i]
            if isinstance(layer, CprGDN):
                o = layer.prefill(slots_t, slots, qkv, a, bb, qsl, prefill_query_start_loc=cu, fuse_l2norm=b.fuse_ops)
                return b.gdn_out(i, o, z)
            if not b.fuse_ops:
                return b.gdn_out(i, layer.prefill(slots_t, slots, qkv, a, bb, qsl, prefill_query_start_loc=cu), z)
            o = layer.prefill(slots_t, slots, qkv, a, bb, qsl, prefill_query_start_loc=cu,
                              gated_norm=b.gdn_gated_norm(i, z))
            return b.gdn_out(i, o, z, normed=True)

        x = b.run_layers(b.embed(tokens), mixer)
        for s, n in zip(slots, lens):
            self.context[s] = n
        return x.index_select(0, torch.from_numpy(offs[1:].astype(np.int64) - 1).to(dev))

    def _decode_state(self, slots: list):
        """Device-resident description of a decode batch: slot ids, each sequence's context length
        (advanced on the device after every step) and where its keys start."""
        dev = self.blocks.w.embed.device
        n = len(slots)
        ctx = np.array([self.context[s] for s in slots], dtype=np.int32)
        rows = np.array([self.kv_rows[s] for s in slots], dtype=np.int64)
        return {
            "slots": list(slots),
            "slots_t": torch.tensor(slots, dtype=torch.int64, device=dev),
            "ctx": torch.from_numpy(ctx).to(dev),
            "kv_start": torch.from_numpy(rows * self.max_len).to(dev),
            "cu": torch.arange(n + 1, dtype=torch.int32, device=dev),
        }

    def _decode_device(self, st: dict, tokens: torch.Tensor) -> torch.Tensor:
        """One decode step from device tensors only (no host read, fixed shapes): what a captured graph
        replays. Advances ``st["ctx"]`` in place."""
        b, c = self.blocks, self.cfg
        positions, kv_start, cu, slots_t = st["ctx"], st["kv_start"], st["cu"], st["slots_t"]
        kv_index = kv_start + positions

        def mixer(i, x):
            if c.is_attention(i):
                q, k, v = b.attn_qkv(i, x, positions)
                self.kv[i].write(kv_index, k, v)
                kf, vf = self.kv[i].flat()
                return b.attn_out(i, varlen_attention(q, kf, vf, cu, 1, kv_start=kv_start, q_pos0=positions))
            qkv, z, bb, a = b.gdn_in(i, x)
            return b.gdn_out(i, self.gdn[i].decode(slots_t, qkv, a, bb), z)

        x = b.run_layers(b.embed(tokens), mixer)
        positions += 1
        return x

    @torch.no_grad()
    def decode(self, slots: list, tokens: torch.Tensor) -> torch.Tensor:
        """Feed one token per sequence; returns the final-normed hidden states ``[N, H]``."""
        if max(self.context[s] for s in slots) >= self.max_len:
            raise RuntimeError(f"[isoexec-amd] a sequence reached the cache length {self.max_len}")
        x = self._decode_device(self._decode_state(slots), tokens)
        for s in slots:
            self.context[s] += 1
        return x

    @torch.no_grad()
    def capture_decode(self, slots: list) -> "DecodeGraph":
        """Record one decode step for this fixed batch as a HIP graph. The sequences must already hold
        state (prefill, and one eager decode step so that every kernel has been launched once)."""
        return DecodeGraph(self, slots)

    @torch.no_grad()
    def generate(self, slots: list, prompts: torch.Tensor, prompt_lens: list, steps: int, *, seed: int = 0,
                 full_row_logprobs=None, use_graph: bool = False):
        """Sample ``steps`` tokens per sequence (Gumbel-max over the logits, seeded) and record each
        sampled token's logprob as the engine reports it. ``full_row_logprobs(logits) -> [N, V] fp32``
        is the engine's logprob producer (default: the row-invariant full-row entry). Returns
        ``(tokens [N, steps] int64, logprobs [N, steps] fp32)``."""
        from ..ops.logprobs.rowinv import full_forward

        if full_row_logprobs is None:
            full_row_logprobs = lambda logits: full_forward(logits, leaves())
        dev = prompts.device
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        x = self.prefill(slots, prompts, prompt_lens)
        out_tok, out_lp = [], []
        for step in range(steps):
            logits = self.blocks.logits(x)
            lp_rows = full_row_logprobs(logits)
            u = torch.rand(logits.shape, generator=g, device=dev).clamp_(min=1e-20)
            tok = (logits.float() - torch.log(-torch.log(u))).argmax(dim=-1)
            out_tok.append(tok)
            out_lp.append(lp_rows.gather(1, tok.unsqueeze(1)).squeeze(1))
            if step + 1 < steps:
                if use_graph and step >= 1:
                    if step == 1:
                        graph = self.capture_decode(slots)
                    x = graph.step(tok)
                else:
                    x = self.decode(slots, tok)
        return torch.stack(out_tok, dim=1), torch.stack(out_lp, dim=1)


class DecodeGraph:
    """One decode step of a fixed batch, captured once and replayed.

    A decode step is ~45 small launches per layer; at batch 64 their launch cost is about half the step.
    The step reads nothing on the host and every shape is fixed, so the whole step is recorded into one
    HIP graph: the token ids live in a static input tensor, each sequence's position in a device counter
    the graph itself advances, and the output in a static tensor the caller must consume before the next
    replay. Replays run the same kernels on the same data as the eager step, so the bits are identical.
    Nothing that clears memory is recorded (outputs are fully overwritten).
    """

    def __init__(self, engine: RolloutEngine, slots: list):
        self.engine, self.slots = engine, list(slots)
        self.state = engine._decode_state(slots)
        dev = self.state["ctx"].device
        self.tokens = torch.zeros(len(slots), dtype=torch.int64, device=dev)
        for layer in engine.gdn.values():
            layer.flush_slot_map()  # the slot map is read, never written, inside the graph
        self.graph = torch.cuda.CUDAGraph()
        saved = self.state["ctx"].clone()
        with torch.cuda.graph(self.graph):
            self.out = engine._decode_device(self.state, self.tokens)
        # Capture records without running, but the position counter update was traced on the real
        # tensor: restore it in case the backend executed anything eagerly.
        self.state["ctx"].copy_(saved)

    @torch.no_grad()
    def step(self, tokens: torch.Tensor) -> torch.Tensor:
        eng = self.engine
        if max(eng.context[s] for s in self.slots) >= eng.max_len:
            raise RuntimeError(f"[isoexec-amd] a sequence reached the cache length {eng.max_len}")
        self.tokens.copy_(tokens)
        self.graph.replay()
        for s in self.slots:
            eng.context[s] += 1
        return self.out
