"""One GatedDeltaNet layer's engine-side core: owned state pools behind a slot -> row table.

Reference: isoexec/ops/gdn/gdn_recurrent_state.py:120-869 (``RecurrentGDN``). The engine names a
request by a slot id drawn from a space far larger than the number of live requests, so the recurrent
(fp32) and convolution (bf16) states live in pools of ``capacity + 1`` rows and a table maps slot ids
to rows. Row 0 is the null row: it is never handed out, unknown slots and padded lanes resolve to
it, and every kernel skips a row index <= 0.

The bookkeeping is split from the device work:

* ``SlotTable`` is pure host code -- the slot <-> row maps, the free list, eviction order and the
  outbox of pending device-map edits. It touches no tensor, so it is tested without a device.
* ``RecurrentGDN`` owns the pools and the device mirror of the table, and runs prefill and decode.
  Prefill is one packed convolution launch, two l2norms, one gate and one scan for the whole batch;
  a sequence's state row is named once (loaded before its first token, stored after its last), so no
  ``[N, Tmax]`` index map is built. Decode is host-free: the slot lookup, the in-pool convolution
  window slide and the scan all run from device tensors of fixed shape.
"""

from __future__ import annotations

import os
from collections import OrderedDict
from typing import Callable, Iterable, Sequence

import numpy as np
import torch

from .gdn_ops import conv_packed, decode_prep, gate_and_beta_fp32, gdn_l2norm, gdn_recurrent_kernel

_SLOT_MAP_ENV = "SKYRL_ISOEXEC_GDN_SLOT_MAP_SIZE"
_CHUNKED_PREFILL_ENV = "SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL"
_NATIVE_STATE_ENV = "SKYRL_ISOEXEC_GDN_NATIVE_STATE"
_OFF = ("", "0", "false", "no")

# How often the eviction path had to read the device's last-used clock back to the host.
_HOST_BOOKKEEPING_STATS = {"lru_device_fallback": 0}


def _slot_map_size() -> int:
    """Entries in the slot -> row map. Read at construction: the tensor is never reallocated."""
    return int(os.environ.get(_SLOT_MAP_ENV) or 65536)


def chunked_prefill_enabled() -> bool:
    """True when a prefill whose slot already holds a row resumes from that row's state."""
    return os.environ.get(_CHUNKED_PREFILL_ENV, "0").lower() not in _OFF


def native_state_enabled() -> bool:
    """True when the state should live in tensors the engine owns, indexed by block id."""
    return os.environ.get(_NATIVE_STATE_ENV, "0").lower() not in _OFF


class SlotTable:
    """Which pool row each live slot owns. Host-only.

    Invariants, checked on every mutation: a row has at most one owner, a free row has none, and the
    two directions of the map agree. A violated invariant raises: it would alias two requests' states.
    """

    def __init__(self, capacity: int, map_size: int, *, driver_managed: bool = False):
        if capacity < 1:
            raise ValueError(f"capacity must be >= 1, got {capacity}")
        self.capacity = int(capacity)
        self.map_size = int(map_size)
        self.driver_managed = bool(driver_managed)
        self.row_of: "OrderedDict[int, int]" = OrderedDict()
        self.slot_of: dict[int, int] = {}
        self.free: list[int] = list(range(1, capacity + 1))
        self._free_set: set[int] = set(self.free)
        self.outbox: dict[int, int] = {}

    # -- queries
    def holds(self, slot: int) -> bool:
        return int(slot) in self.row_of

    def __len__(self) -> int:
        return len(self.row_of)

    def require_row(self, slot: int) -> int:
        """The row of a slot known to belong to a live request. A miss is unrecoverable: the device
        path would fold the lane onto the null row and share one state across requests."""
        row = self.row_of.get(int(slot))
        if row is None:
            raise RuntimeError(
                f"[isoexec-gdn] LIVE state slot {int(slot)} has no mapped row (host map holds "
                f"{len(self.row_of)} entries; device map {self.map_size} slots; capacity={self.capacity}). "
                f"Decode would fold this lane onto null row 0. Causes: a slot-id space the bookkeeping never "
                f"mapped, a block id past the map (raise {_SLOT_MAP_ENV}), or a row evicted while its request lived."
            )
        return row

    def check(self) -> None:
        if len(self.slot_of) != len(self.row_of):
            raise RuntimeError("[isoexec-gdn] a recurrent row is also mapped by a second slot, or the table was edited outside its methods")
        if len(self._free_set) != len(self.free):
            raise RuntimeError("[isoexec-gdn] free-list rows contain a duplicate, or the free list was edited outside its methods")

    # -- mutations
    def _bind(self, slot: int, row: int) -> None:
        owner = self.slot_of.get(row)
        if owner is not None:
            raise RuntimeError(f"[isoexec-gdn] recurrent row {row} is already owned by slot {owner}; assigning slot {slot} would alias live states")
        if row in self._free_set:
            raise RuntimeError(f"[isoexec-gdn] row {row} is on the free list and cannot be bound")
        self.row_of[slot] = row
        self.slot_of[row] = slot
        self.outbox[slot] = row

    def _unbind(self, slot: int) -> int:
        row = self.row_of.pop(slot)
        owner = self.slot_of.pop(row, None)
        if owner != slot:
            raise RuntimeError(f"[isoexec-gdn] recurrent row {row} is also mapped or owned by slot {owner}, not slot {slot}")
        return row

    def assign_many(self, slots: Sequence[int], lru_snapshot: Callable[[], Sequence[int]] | None = None) -> list[int]:
        """Rows for a prefill batch, in order. A slot that already holds a row keeps it (and becomes
        most recent); otherwise a free row is taken; with none free, the least recently used row not
        claimed by this batch is evicted. ``lru_snapshot()`` returns ``last_used`` per row and is
        called at most once per batch: re-reading it between evictions could hand one row out twice.
        """
        want = [int(s) for s in slots]
        if not want:
            return []
        self.check()
        bad = [s for s in want if s < 0 or s >= self.map_size]
        if bad:
            raise RuntimeError(
                f"[isoexec-gdn] state slot {bad[0]} exceeds the slot map ({self.map_size}). Raise {_SLOT_MAP_ENV}; "
                f"the map cannot grow because replayed launches hold its address."
            )
        newcomers = {s for s in want if s not in self.row_of}
        if self.driver_managed and len(newcomers) > len(self.free):
            # Refuse the whole batch before touching anything: exhaustion must not leave a half-edited table.
            raise RuntimeError(
                f"[isoexec-gdn] driver-managed state pool exhausted: capacity={self.capacity}, mapped={len(self.row_of)}, "
                f"free={len(self.free)}, missing={len(newcomers)} while assigning {len(want)} prefill slots. Every mapped "
                f"row is lifecycle-owned, so none may be evicted; finished requests must be released first."
            )
        rows: list[int] = []
        claimed: set[int] = set()
        order: list[int] | None = None
        cursor = 0
        for s in want:
            if s in self.row_of:
                row = self._unbind(s)
            elif self.free:
                row = self.free.pop()
                self._free_set.remove(row)
            else:
                if order is None:
                    if lru_snapshot is None:
                        raise RuntimeError("[isoexec-gdn] state pool is full and no eviction order is available")
                    used = list(lru_snapshot())
                    _HOST_BOOKKEEPING_STATS["lru_device_fallback"] += 1
                    order = sorted(range(1, len(used)), key=lambda r: (used[r], r))
                while cursor < len(order) and order[cursor] in claimed:
                    cursor += 1
                if cursor >= len(order):
                    raise RuntimeError(
                        f"[isoexec-gdn] prefill batch of {len(want)} slots exceeds the {len(order)} evictable state rows in "
                        f"this pool: every row is already claimed by THIS batch, so an eviction would hand one row to two "
                        f"live requests."
                    )
                row = order[cursor]
                cursor += 1
                victim = self.slot_of.get(row)
                if victim is not None:
                    self._unbind(victim)
                    self.outbox[victim] = 0
            self._bind(s, row)
            claimed.add(row)
            rows.append(row)
        self.check()
        return rows

    def release(self, slot: int) -> int | None:
        """Return a finished request's row to the free list; the freed row, or None if it held none."""
        slot = int(slot)
        if slot not in self.row_of:
            return None
        row = self._unbind(slot)
        if row in self._free_set:
            raise RuntimeError(f"[isoexec-gdn] released row {row} is already on the free list")
        if 0 <= slot < self.map_size:
            self.outbox[slot] = 0
        self.free.append(row)
        self._free_set.add(row)
        self.check()
        return row

    def release_all(self) -> list[int]:
        return [row for row in (self.release(s) for s in list(self.row_of)) if row is not None]

    def rebind(self, old: int, new: int) -> int | None:
        """Rename a live request's slot. The row and its state do not move; whatever ``new`` held
        belonged to a finished request and is released. Returns that released row, if any."""
        old, new = int(old), int(new)
        if old == new or old not in self.row_of:
            return None
        if not 0 <= new < self.map_size:
            raise RuntimeError(f"[isoexec-gdn] cannot rebind onto slot {new}: outside the slot map ({self.map_size})")
        row = self._unbind(old)
        if 0 <= old < self.map_size:
            self.outbox[old] = 0
        dropped = self.release(new)
        self._bind(new, row)
        self.check()
        return dropped

    def drain_outbox(self):
        """Pending device-map edits as ``(slots, rows)`` int64 arrays, or None; clears the outbox."""
        n = len(self.outbox)
        if n == 0:
            return None
        keys = np.fromiter(self.outbox.keys(), dtype=np.int64, count=n)
        vals = np.fromiter(self.outbox.values(), dtype=np.int64, count=n)
        self.outbox.clear()
        return keys, vals


def build_recurrent_gdn(*, max_num_seqs: int, ssm_state=None, conv_state=None, **kw) -> "RecurrentGDN":
    """A ``RecurrentGDN`` sized by the scheduler's concurrency cap. ``ssm_state`` / ``conv_state``
    (both or neither) hand the layer engine-owned state tensors instead of private pools."""
    return RecurrentGDN(capacity=max_num_seqs, ssm_state=ssm_state, conv_state=conv_state, **kw)


def flush_slot_maps(layers: Iterable["RecurrentGDN"]) -> int:
    """Flush every layer's outbox. Returns the number of edits applied."""
    return sum(layer.flush_slot_map() for layer in layers)


def invalidate_all_states(layers: Iterable["RecurrentGDN"]) -> int:
    """The weight-sync / sleep-wake hook: every request's state was computed under weights that no
    longer exist, so every row is released and both pools are zeroed. Returns the rows released."""
    freed = 0
    for layer in layers:
        freed += layer.reset()
    return freed


class RecurrentGDN:
    def __init__(
        self,
        *,
        capacity: int,
        conv_weight: torch.Tensor,  # [D, W]
        conv_bias: torch.Tensor | None,
        A_log: torch.Tensor,  # [HV]
        dt_bias: torch.Tensor,  # [HV]
        num_k_heads: int,
        head_k_dim: int,
        num_v_heads: int,
        head_v_dim: int,
        activation: str | None = "silu",
        dtype: torch.dtype = torch.bfloat16,
        device: torch.device | str = "cuda",
        ssm_state: torch.Tensor | None = None,
        conv_state: torch.Tensor | None = None,
        slot_map_hint: int = 0,
        driver_managed: bool = False,
    ):
        if num_v_heads % num_k_heads:
            raise ValueError(f"num_v_heads {num_v_heads} must be a multiple of num_k_heads {num_k_heads}")
        W = conv_weight.shape[-1]
        D = 2 * num_k_heads * head_k_dim + num_v_heads * head_v_dim
        if conv_weight.shape[0] != D:
            raise ValueError(f"conv_weight has {conv_weight.shape[0]} channels, the head layout needs {D}")
        self.capacity = capacity
        self._native = ssm_state is not None or conv_state is not None
        if self._native:
            if ssm_state is None or conv_state is None:
                raise ValueError("[isoexec-gdn] native state needs BOTH ssm_state and conv_state")
            # bf16 would round the state at every step and break the prefill -> decode round trip.
            if ssm_state.dtype != torch.float32:
                raise RuntimeError(
                    f"[isoexec-gdn] native ssm state resolved to {ssm_state.dtype}, not float32. "
                    "Set mamba_ssm_cache_dtype=float32 at engine build."
                )
            if conv_state.shape[-1] != W - 1 or conv_state.shape[-2] != D:
                raise RuntimeError(
                    f"[isoexec-gdn] native conv_state {tuple(conv_state.shape)} is not (num_blocks, {D}, {W - 1}); "
                    "the orientation is wrong (transpose it before handing it over)."
                )
            if not ssm_state.is_contiguous() or not conv_state.is_contiguous():
                raise RuntimeError("[isoexec-gdn] native state tensors must be contiguous")
            self.ssm_state, self.conv_state = ssm_state, conv_state
            self.table = None
        else:
            rows = capacity + 1
            self.ssm_state = torch.zeros(rows, num_v_heads, head_v_dim, head_k_dim, dtype=torch.float32, device=device)
            self.conv_state = torch.zeros(rows, D, W - 1, dtype=dtype, device=device)
            self.table = SlotTable(capacity, max(_slot_map_size(), int(slot_map_hint)), driver_managed=driver_managed)
            # Device mirror of the table, the per-row last-use tick and the clock it is stamped from.
            # All three keep their addresses for the life of the layer.
            self.slot2row = torch.zeros(self.table.map_size, dtype=torch.long, device=device)
            self.last_used = torch.zeros(rows, dtype=torch.long, device=device)
            self._clock = torch.zeros((), dtype=torch.long, device=device)
        self.conv_weight = conv_weight.contiguous()
        self.conv_bias = None if conv_bias is None else conv_bias.contiguous()
        self.A_log, self.dt_bias = A_log.float().contiguous(), dt_bias.float().contiguous()
        self.num_k_heads, self.head_k_dim = num_k_heads, head_k_dim
        self.num_v_heads, self.head_v_dim = num_v_heads, head_v_dim
        self.activation = activation
        self.fused_decode_prep = True   # False: the decode step takes conv, l2norm and gating as separate launches
        self._decode_cu: dict[int, torch.Tensor] = {}

    # -- table passthroughs (the reference's method names)
    @property
    def _slot2row(self):
        return self.table.row_of if self.table is not None else {}

    @property
    def _driver_managed(self) -> bool:
        return bool(self.table and self.table.driver_managed)

    def _assign(self, slot: int) -> int:
        return self._assign_many((slot,))[0]

    def _assign_many(self, slots) -> list[int]:
        rows = self.table.assign_many(slots, lru_snapshot=self.last_used.tolist)
        self.flush_slot_map()
        # One clock scatter for the batch; a row named twice keeps its last tick.
        ticks = {r: j + 1 for j, r in enumerate(rows)}
        if ticks:
            buf = np.array([list(ticks.keys()), list(ticks.values())], dtype=np.int64)
            t = torch.from_numpy(buf).to(self.last_used.device, non_blocking=True)
            self.last_used[t[0]] = self._clock + t[1]
            self._clock += len(rows)
        return rows

    def flush_slot_map(self) -> int:
        """Push pending slot-map edits to the device in one scatter. Must run before any device read
        of the map and never inside a captured region."""
        if self._native:
            return 0
        pending = self.table.drain_outbox()
        if pending is None:
            return 0
        keys, vals = pending
        t = torch.from_numpy(np.stack([keys, vals])).to(self.slot2row.device, non_blocking=True)
        self.slot2row[t[0]] = t[1]
        return len(keys)

    def release_slot(self, slot: int) -> int | None:
        if self._native:
            return None
        row = self.table.release(slot)
        if row is not None:
            self._on_row_released(row)
        return row

    def require_row(self, slot: int) -> int:
        if self._native:
            return int(slot)
        return self.table.require_row(slot)

    def rebind_slot(self, old: int, new: int) -> None:
        if self._native:
            return
        dropped = self.table.rebind(old, new)
        if dropped is not None:
            self._on_row_released(dropped)

    def _on_row_released(self, row: int) -> None:
        """Hook for a subclass that keeps side state per row."""

    def reset(self) -> int:
        """Release every row and zero both pools. Returns the number of rows released."""
        freed = 0
        if not self._native:
            freed = len(self.table.release_all())
            self.flush_slot_map()
            self.last_used.zero_()
            self._clock.zero_()
        self.ssm_state.zero_()
        self.conv_state.zero_()
        return freed

    # -- device helpers
    def _rows(self, slots: torch.Tensor) -> torch.Tensor:
        """Slot ids -> pool rows on the device, branch-free. Ids outside the map (padding carries
        arbitrary values) are clamped into it, and unknown ids read row 0."""
        s = slots.long()
        if self._native:
            blocks = self.ssm_state.shape[0]
            return torch.where(s < blocks, s, torch.zeros_like(s)).clamp_(min=0)
        return self.slot2row[s.clamp(0, self.slot2row.numel() - 1)]

    def _rows_pair(self, slots: torch.Tensor):
        """``(rows int64, rows int32)``: one launch when the fused resolver serves the arguments
        (gdn_recurrent_state.py:286-299), else the eager chain."""
        if not self._native:
            from .gdn_cpr_rows import cpr_resolve_rows, fused_rows_enabled

            if fused_rows_enabled() and slots.is_cuda:
                pair = cpr_resolve_rows(slots, self.slot2row)
                if pair is not None:
                    return pair
        rows = self._rows(slots)
        return rows, rows.to(torch.int32)

    def _decode_rows(self, slots: torch.Tensor) -> torch.Tensor:
        """int32 rows of a decode batch, with the rows' use stamp advanced (private pool only). One launch when
        the fused resolver serves the arguments."""
        from .gdn_cpr_rows import fused_rows_enabled, resolve_and_stamp

        if fused_rows_enabled() and slots.is_cuda:
            if self._native:
                rows32 = resolve_and_stamp(slots, blocks=self.ssm_state.shape[0])
            else:
                rows32 = resolve_and_stamp(slots, slot2row=self.slot2row, last_used=self.last_used, clock=self._clock)
            if rows32 is not None:
                return rows32
        rows, rows32 = self._rows_pair(slots)
        if not self._native:
            self._clock += 1
            self.last_used[rows] = self._clock
        return rows32

    def _split_qkv_raw(self, y: torch.Tensor):
        """Post-conv ``[T, D]`` -> views ``q, k [T, H, K]`` and ``v [T, HV, V]`` (token pitch D, no copy)."""
        T = y.shape[0]
        kd = self.num_k_heads * self.head_k_dim
        q = y[:, :kd].unflatten(1, (self.num_k_heads, self.head_k_dim))
        k = y[:, kd : 2 * kd].unflatten(1, (self.num_k_heads, self.head_k_dim))
        v = y[:, 2 * kd :].unflatten(1, (self.num_v_heads, self.head_v_dim))
        return q, k, v

    def _split_qkv(self, y: torch.Tensor):
        """As ``_split_qkv_raw`` with q and k L2-normalised. Heads stay GQA-compressed: the scan maps
        value head hv to key head ``hv // (HV / H)`` itself."""
        q, k, v = self._split_qkv_raw(y)
        if y.ndim == 2 and y.stride(1) == 1:
            # q and k are adjacent column blocks of y: one launch normalises the 2H rows of each token
            H = self.num_k_heads
            qk = gdn_l2norm(y[:, : 2 * H * self.head_k_dim].unflatten(1, (2 * H, self.head_k_dim)))
            return qk[:, :H], qk[:, H:], v
        return gdn_l2norm(q), gdn_l2norm(k), v

    def _gate_and_beta(self, a: torch.Tensor, b: torch.Tensor):
        return gate_and_beta_fp32(a, b, self.A_log, self.dt_bias)

    def _continuation_mask(self, slots_cpu, has_initial_state) -> list[bool]:
        """Which prefill rows resume carried state. Table membership and the scheduler's
        ``has_initial_state`` must agree: membership alone would mistake a reissued slot id for a
        continuation. ``None`` means the caller has no opinion, and membership decides."""
        resume = chunked_prefill_enabled()
        held = [self.table.holds(s) for s in slots_cpu]
        if has_initial_state is None:
            return [resume and h for h in held]
        raw = has_initial_state if isinstance(has_initial_state, (list, tuple)) else has_initial_state.tolist()
        want = [bool(v) for v in raw]
        for i, (w, h) in enumerate(zip(want, held)):
            if w and not h:
                raise RuntimeError(
                    f"[isoexec-gdn] the scheduler reports an initial state for prefill row {i} (slot {int(slots_cpu[i])}) "
                    f"but the private state pool holds none -- a prefix-cache hit. A private pool cannot resume a prefix "
                    f"it did not itself scan."
                )
        return [resume and w and h for w, h in zip(want, held)]

    # -- public API
    @torch.no_grad()
    def prefill(
        self,
        slots: torch.Tensor,  # [N] device slot ids
        slots_cpu: list,
        x: torch.Tensor,  # [T, D] packed, pre-conv
        a: torch.Tensor,  # [T, HV]
        b: torch.Tensor,  # [T, HV]
        qsl: list,  # [N+1] token offsets into the packed region
        has_initial_state=None,
        prefill_query_start_loc: torch.Tensor | None = None,
        gated_norm: tuple | None = None,
    ) -> torch.Tensor:
        """Prefill a packed batch of N prompts (or prompt chunks). Returns ``o [T, HV, V]``; with ``gated_norm``
        (``gdn_recurrent_kernel``'s) the output comes back through the layer's gated output norm."""
        rows, is_cont, rows_out, cu, q, k, v, g, beta = self._prefill_prepare(
            slots_cpu, x, a, b, qsl, has_initial_state, prefill_query_start_loc, fuse_l2norm=gated_norm is not None)
        o = gdn_recurrent_kernel(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), g.unsqueeze(0), beta.unsqueeze(0),
                                 ssm_state=self.ssm_state, state_indices=rows_out, cu_seqlens=cu, gated_norm=gated_norm)
        return o[0]

    def _prefill_prepare(self, slots_cpu, x, a, b, qsl, has_initial_state, prefill_query_start_loc, fuse_l2norm=True):
        """Everything of a prefill in front of the scan: rows assigned (fresh rows zeroed), the convolution with
        its window carried in the pool, q/k normalised, gate and beta. Returns ``(rows, is_cont, rows_out int32
        device, cu int32 device, q, k, v, g, beta)`` with q, k ``[T, H, K]``, v ``[T, HV, V]``, g, beta ``[T, HV]``."""
        N = len(slots_cpu)
        dev = x.device
        if len(qsl) != N + 1 or qsl[-1] != x.shape[0]:
            raise ValueError(f"qsl {list(qsl)} does not describe {N} sequences over {x.shape[0]} packed tokens")
        if self._native:
            rows = [int(s) for s in slots_cpu]
            blocks = self.ssm_state.shape[0]
            bad = [r for r in rows if r < 0 or r >= blocks]
            if bad:
                raise RuntimeError(f"[isoexec-gdn] NATIVE prefill: block id(s) {bad[:8]} out of range for a state tensor with {blocks} rows")
            if has_initial_state is None:
                is_cont = [False] * N
            else:
                raw = has_initial_state if isinstance(has_initial_state, (list, tuple)) else has_initial_state.tolist()
                is_cont = [bool(v) for v in raw]
        else:
            # Membership is read before assignment edits the table; fresh and resumed rows may mix.
            is_cont = self._continuation_mask(slots_cpu, has_initial_state)
            rows = self._assign_many(slots_cpu)
        # One upload carries the three row lists: where each sequence stores, where it resumes from
        # (0 = from nothing) and which rows start fresh (0 = none; zeroing the null row is harmless).
        meta = np.array(
            [rows, [r if c else 0 for r, c in zip(rows, is_cont)], [0 if c else r for r, c in zip(rows, is_cont)]],
            dtype=np.int32,
        )
        meta_t = torch.from_numpy(meta).to(dev, non_blocking=True)
        rows_out, rows_in = meta_t[0], meta_t[1]
        cu = prefill_query_start_loc
        if cu is None:
            cu = torch.from_numpy(np.asarray(qsl, dtype=np.int32)).to(dev, non_blocking=True)
        # A fresh row must start from zero; a resumed row keeps what the previous chunk left.
        self._zero_fresh_rows(meta_t[2].long())
        if fuse_l2norm:  # q and k leave the convolution's launch normalised where the library serves that form
            y = conv_packed(x, self.conv_weight, self.conv_bias, cu_seqlens=cu, conv_state=self.conv_state,
                            rows_in=rows_in, rows_out=rows_out, activation=self.activation,
                            l2norm_qk=2 * self.num_k_heads * self.head_k_dim, head_k_dim=self.head_k_dim)
            q, k, v = self._split_qkv_raw(y)
        else:  # the two ops apart (what a traced run asks for: each door's output is its own region)
            y = conv_packed(x, self.conv_weight, self.conv_bias, cu_seqlens=cu, conv_state=self.conv_state,
                            rows_in=rows_in, rows_out=rows_out, activation=self.activation)
            q, k, v = self._split_qkv(y)
        g, beta = self._gate_and_beta(a, b)
        return rows, is_cont, rows_out, cu, q, k, v, g, beta

    def _zero_fresh_rows(self, fresh_rows: torch.Tensor) -> None:
        """Rows that start a new request (device int64, 0 = none)."""
        self.ssm_state.index_fill_(0, fresh_rows, 0.0)

    def _decode_prepare(self, x, a, b, rows32, cu):
        """A decode step in front of its scan: the convolution on the row's W-1 stored inputs (the window slides in
        the pool itself), q and k normalised, gate and beta. One launch where the library serves the shape
        (``decode_prep``), else the three launches it stands for: the same bits either way."""
        fused = None
        if self.fused_decode_prep and a.ndim == 2 and b.ndim == 2:
            fused = decode_prep(x, a, b, self.conv_weight, self.conv_bias, self.A_log, self.dt_bias, self.conv_state, rows32,
                                H=self.num_k_heads, K=self.head_k_dim, HV=self.num_v_heads, V=self.head_v_dim,
                                activation=self.activation)
        if fused is not None:
            y, g, beta = fused
            q, k, v = self._split_qkv_raw(y)
            return q, k, v, g, beta
        y = conv_packed(x, self.conv_weight, self.conv_bias, cu_seqlens=cu, conv_state=self.conv_state,
                        rows_in=rows32, rows_out=rows32, activation=self.activation)
        q, k, v = self._split_qkv(y)
        g, beta = self._gate_and_beta(a, b)
        return q, k, v, g, beta

    @torch.no_grad()
    def decode(self, slots: torch.Tensor, x: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """One decode step for N requests: ``x [N, D]`` pre-conv, ``a, b [N, HV]``. Returns
        ``o [N, HV, V]``. Host-free and shape-static. A padded lane resolves to row 0: it reads a zero
        convolution history, writes no state and returns zeros."""
        N = x.shape[0]
        rows32 = self._decode_rows(slots)
        cu = self._decode_cu.get(N)
        if cu is None:
            cu = self._decode_cu[N] = torch.arange(N + 1, dtype=torch.int32, device=x.device)
        q, k, v, g, beta = self._decode_prepare(x, a, b, rows32, cu)
        o = gdn_recurrent_kernel(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), g.unsqueeze(0), beta.unsqueeze(0),
                                 ssm_state=self.ssm_state, state_indices=rows32, cu_seqlens=cu, time_tile=1)
        return o[0]
