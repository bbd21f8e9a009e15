"""Engine state for the boundary (cpr) form of the GatedDeltaNet layer (reference: ops/gdn/gdn_cpr_state.py:379-1245).

``CprGDN`` is ``RecurrentGDN`` plus, per pool row: the fp32 ENTRY state (the unrounded chain at the last chunk
boundary), open-chunk buffers holding the prepared k, v, g, beta of the tokens since that boundary, and the absolute
position. The running state (``ssm_state``) is what a token is scanned from: at a boundary it is the entry state
snapshotted in the wire dtype, inside a chunk it advances token by token. That makes prefill + decode reproduce
``gdn_cpr_fwd`` bit for bit however the tokens are cut into calls:

* decode: one recurrent step from the running state, the token appended to the row's buffers (one launch), and for
  rows whose position reached a multiple of C the boundary pass: a state-only scan over the row's C buffered tokens
  from its entry state (the same recurrence, so the chain is the one a single long scan would produce), then
  running <- snapshot(entry). The due rows are marked on the device, the boundary scan runs over the whole pool with
  every other row a null lane, so the step reads nothing on the host and can be replayed from a HIP graph.
* prefill: a chain pass over [buffered tokens ++ new tokens up to the last boundary crossed] with the state stored
  at every boundary, then one segmented scan of the new tokens (first segment from the running state, the others
  from the boundary snapshots), then the tail of the open chunk goes to the buffers.

Around that state, as in the reference:

* the boundary store (``CprBoundaryStore``, gdn_cpr_state.py:96-196): at a multiple of C a request's whole state is
  (fp32 entry state, convolution window), so a prefix that ends on a boundary can be resumed from a stored pair and
  the continuation is the ordinary chunked-prefill one -- bit for bit what a cold prefill of the whole prompt gives.
  Prefill stashes the pairs of the last boundaries it closes (``_apc_pending``), ``cpr_apc_publish`` stacks them over
  the layers and stores them under the driver's prefix key, ``cpr_apc_adopt_many`` installs stored pairs for a
  scheduler step. A miss is never a correctness event: the prompt is prefilled cold.
* sleep (gdn_cpr_sleep.py:45-282): every layer's seven state tensors are views into one flat allocation, which
  ``cpr_sleep`` gives back to the device with no host copy and ``cpr_wake`` makes anew, zeroed, with every row released.
  The store is dropped first, so nothing advertises a checkpoint no layer could continue from. With
  ``SKYRL_ISOEXEC_GDN_CPR_SLEEP=1`` (the reference's switch) the allocation is a ``DeviceArena``: a reserved range of
  device addresses whose memory is unmapped at sleep and mapped again at wake (``ix_arena_*``), so the state keeps its
  address and a decode graph captured before the sleep replays after the wake. Without the switch it is an ordinary
  allocation, the wake makes a new one at a new address, and such a graph has to be captured again.

The reference's lazy boundary resync (``host_resync`` / ``layer_batched_resync``, gdn_cpr_state.py:295-358, 581-648)
has no counterpart: it exists to keep a host-side position read out of the captured decode step, and here the boundary
pass runs inside the step from device-side marks.
"""
from __future__ import annotations

import os
import sys
from collections import OrderedDict
from typing import Callable, Optional

import numpy as np
import torch

from ... import _lib
from .gdn_cpr import chunk_boundary_states
from .gdn_ops import gdn_recurrent_kernel
from .gdn_recurrent_state import RecurrentGDN

CPR_LAYERS: list = []

_CPR_APC_ENV = "SKYRL_ISOEXEC_GDN_CPR_APC"
_CPR_APC_MB_ENV = "SKYRL_ISOEXEC_GDN_CPR_APC_MB"
_OFF = ("", "0", "false", "no")
# rows of one prefill call that may stash checkpoints: each stash is a cloned fp32 state held until it is published
_APC_PENDING_MAX = 16
_APC_ADOPT_WRITE_BATCH = 64


def cpr_apc_enabled() -> bool:
    """True when prefill stashes boundary checkpoints for the store (default off; gdn_cpr_state.py:71-73)."""
    return os.environ.get(_CPR_APC_ENV, "0").strip().lower() not in _OFF


def cpr_apc_shared_mode() -> bool:
    """True for ``SKYRL_ISOEXEC_GDN_CPR_APC`` in {2, shm, shared}: the store's membership is mirrored to a scheduler
    in another process, so within an epoch it only grows (a published key must stay servable; :76-83)."""
    return os.environ.get(_CPR_APC_ENV, "0").strip().lower() in ("2", "shm", "shared")


def cpr_apc_budget_bytes() -> int:
    """Device-memory ceiling of the store, ``SKYRL_ISOEXEC_GDN_CPR_APC_MB`` MiB (default 1024; :86-88)."""
    return int(float(os.environ.get(_CPR_APC_MB_ENV, "1024") or 1024) * 2**20)


# Called by ``CprBoundaryStore.clear()`` after the local drop, so that a published index is retracted before anyone can
# be admitted against it. An exception propagates: an index that still advertises dropped entries must not pass silently.
CPR_APC_ON_CLEAR: list = []


def _nbytes(*tensors) -> int:
    return sum(t.numel() * t.element_size() for t in tensors)


class CprBoundaryStore:
    """Checkpoints of requests at chunk boundaries, keyed by a digest of the token prefix, least recently used first
    out. A value is ``(position, entry [L, HV, V, K] fp32, conv [L, D, W-1])``: one pair per GDN layer, stacked.

    The store must not outlive the engine's own prefix cache (it would resume a prefix computed under older
    weights): whoever resets that cache calls ``cpr_apc_reset``."""

    def __init__(self, budget_bytes: int, evict: bool = True, say: Optional[Callable[[str], None]] = None):
        self.budget = int(budget_bytes)
        self.evict = bool(evict)  # False: append-only (shared-index mode), a full store refuses instead of evicting
        self._items: "OrderedDict[bytes, tuple]" = OrderedDict()
        self._bytes = 0
        self.hits = self.misses = self.stores = self.evictions = self.full_refusals = self.oversize_refusals = 0
        self._say = say or (lambda msg: print(msg, file=sys.stderr, flush=True))

    def __contains__(self, key: bytes) -> bool:
        return key in self._items

    def __len__(self) -> int:
        return len(self._items)

    @property
    def nbytes(self) -> int:
        return self._bytes

    def get(self, key: bytes):
        item = self._items.get(key)
        if item is None:
            self.misses += 1
            return None
        self._items.move_to_end(key)
        self.hits += 1
        return item

    def put(self, key: bytes, pos: int, entry: torch.Tensor, conv: torch.Tensor) -> bool:
        """True when a NEW checkpoint was stored (the cue to publish its key); a known key is only refreshed."""
        if key in self._items:
            self._items.move_to_end(key)
            return False
        size = _nbytes(entry, conv)
        if size > self.budget:
            self.oversize_refusals += 1
            if self.oversize_refusals == 1:
                self._say(f"[isoexec-cpr-apc] one boundary checkpoint takes {size / 2**20:.1f} MiB, the whole store "
                          f"{self.budget / 2**20:.1f} MiB: nothing can be stored, no prefix will ever hit. Raise "
                          f"{_CPR_APC_MB_ENV} or set {_CPR_APC_ENV}=0.")
            return False
        if self._bytes + size > self.budget and not self.evict:
            self.full_refusals += 1
            if self.full_refusals == 1:
                self._say(f"[isoexec-cpr-apc] store full at {self._bytes / 2**20:.1f} of {self.budget / 2**20:.1f} MiB "
                          f"({len(self._items)} checkpoints) and append-only: new checkpoints are refused until the "
                          f"next reset. Raise {_CPR_APC_MB_ENV} if this repeats.")
            return False
        while self._bytes + size > self.budget and self._items:
            _, (_, old_entry, old_conv) = self._items.popitem(last=False)
            self._bytes -= _nbytes(old_entry, old_conv)
            self.evictions += 1
        self._items[key] = (int(pos), entry, conv)
        self._bytes += size
        self.stores += 1
        return True

    def clear(self) -> None:
        self._items.clear()
        self._bytes = 0
        for hook in list(CPR_APC_ON_CLEAR):
            hook()

    def stats(self) -> dict:
        return {"entries": len(self._items), "MiB": round(self._bytes / 2**20, 1), "hits": self.hits,
                "misses": self.misses, "stores": self.stores, "evictions": self.evictions,
                "full_refusals": self.full_refusals, "oversize_refusals": self.oversize_refusals}


CPR_APC_STORE: Optional[CprBoundaryStore] = None


def cpr_apc_store() -> CprBoundaryStore:
    """The process's store, made on first use with the budget and mode the environment names."""
    global CPR_APC_STORE
    if CPR_APC_STORE is None:
        CPR_APC_STORE = CprBoundaryStore(cpr_apc_budget_bytes(), evict=not cpr_apc_shared_mode())
    return CPR_APC_STORE


def cpr_apc_reset() -> None:
    """Drop every checkpoint. To be called wherever the engine resets its own prefix cache (a weight sync)."""
    if CPR_APC_STORE is not None:
        CPR_APC_STORE.clear()


def cpr_apc_store_invalidate() -> None:
    """Drop the store because its tensors are about to become unreadable (a sleep). Runs BEFORE the release."""
    cpr_apc_reset()


def cpr_apc_publish(layers: list, items: list) -> list:
    """Move the checkpoints that the layers' last prefill stashed into the store.

    ``items`` are ``(slot, position, prefix_key)`` as the driver knows them (it alone can name a prefix). A checkpoint
    is stored when EVERY layer stashed one for that slot's row at that position; the per-layer pairs are stacked on a
    new first axis. Returns the keys newly stored (what a shared index would advertise). Whatever was stashed and not
    asked for is dropped: a stash lives for one step."""
    if not layers:
        return []
    store = cpr_apc_store()
    fresh = []
    for slot, pos, key in items:
        row = layers[0]._slot2row.get(int(slot))
        if row is None or key in store:
            continue
        found = []
        for ly in layers:
            pair = next(((e, c) for p, e, c in ly._apc_pending.get(ly._slot2row.get(int(slot), -1), ()) if p == int(pos)), None)
            if pair is None:
                break
            found.append(pair)
        if len(found) != len(layers):
            continue
        if store.put(key, int(pos), torch.stack([e for e, _ in found]), torch.stack([c for _, c in found])):
            fresh.append(key)
    for ly in layers:
        ly._apc_pending.clear()
    return fresh


def cpr_apc_adopt_many(layers: list, items: list):
    """Install stored boundary states for one scheduler step: ``items`` are ``(slot, position, prefix_key)`` in
    scheduler order; returns the pool row given to each, or ``None`` when any of them cannot be served (then nothing
    was touched: every condition is checked before the first row changes hands; gdn_cpr_state.py:222-278). After a
    successful call the requests' prefills are ordinary continuations (``has_initial_state`` true)."""
    if not items:
        return []
    if not layers:
        return None
    first = layers[0]
    C = first.chunk_size
    store = cpr_apc_store()
    checkpoints = []
    for _slot, pos, key in items:
        if pos <= 0 or pos % C:
            return None
        got = store.get(key)
        if got is None:
            return None
        at, entry, conv = got
        if at != pos or entry.shape[0] != len(layers) or conv.shape[0] != len(layers):
            return None
        checkpoints.append((entry, conv))
    slots = [int(slot) for slot, _pos, _key in items]
    rows_by_layer = [ly._assign_many(slots) for ly in layers]
    rows = rows_by_layer[0]
    if any(other != rows for other in rows_by_layer[1:]):
        raise RuntimeError("[isoexec-gdn] adoption found the layers' state pools out of step: the same request would "
                           "sit in different rows of different layers")
    dev = first.ssm_state.device
    positions = [int(pos) for _slot, pos, _key in items]
    for j, ly in enumerate(layers):
        wire = ly.k_buf.dtype if getattr(ly, "k_buf", None) is not None else torch.bfloat16
        for lo in range(0, len(items), _APC_ADOPT_WRITE_BATCH):
            hi = min(lo + _APC_ADOPT_WRITE_BATCH, len(items))
            r = torch.tensor(rows[lo:hi], dtype=torch.long, device=dev)
            entry = torch.stack([checkpoints[i][0][j] for i in range(lo, hi)])
            conv = torch.stack([checkpoints[i][1][j] for i in range(lo, hi)])
            ly.entry_state[r] = entry
            ly.ssm_state[r] = entry.to(wire).to(torch.float32)   # the running state at a boundary is the snapshot
            ly.conv_state[r] = conv.to(ly.conv_state.dtype)
        ly.pos[torch.tensor(rows, dtype=torch.long, device=dev)] = torch.tensor(positions, dtype=torch.long, device=dev)
        for row in rows:
            ly._apc_pending.pop(row, None)
    return rows


def cpr_apc_adopt(layers: list, slot: int, pos: int, key: bytes) -> bool:
    """One request's adoption; False means a cold prefill (gdn_cpr_state.py:281-287)."""
    return cpr_apc_adopt_many(layers, [(int(slot), int(pos), key)]) is not None


def cpr_arena_specs(*, rows, C, HV, K, V, Hk, dt, gdt, conv_shape) -> list:
    """``[(attribute, shape, dtype), ...]`` of a layer's device state in allocation order (gdn_cpr_state.py:360-371)."""
    return [("ssm_state", (rows, HV, V, K), torch.float32), ("conv_state", tuple(conv_shape), dt),
            ("entry_state", (rows, HV, V, K), torch.float32), ("k_buf", (rows, C, Hk, K), dt),
            ("v_buf", (rows, C, HV, V), dt), ("g_buf", (rows, C, HV), gdt), ("b_buf", (rows, C, HV), dt)]


_CPR_SLEEP_ENV = "SKYRL_ISOEXEC_GDN_CPR_SLEEP"


def cpr_sleep_enabled() -> bool:
    """True when the layers' state lives in an arena that keeps its address over a sleep (gdn_cpr_sleep.py:28-30)."""
    return os.environ.get(_CPR_SLEEP_ENV, "0").strip().lower() not in _OFF


class DeviceArena:
    """A reserved range of device addresses; its memory can be released and restored (zeroed) in place."""

    def __init__(self, nbytes: int, device):
        self.device = torch.device(device)
        handle = _lib.ctypes.c_void_p()
        with torch.cuda.device(self.device):
            rc = _lib.check(_lib.lib().ix_arena_create(int(nbytes), _lib.ctypes.byref(handle),
                                                       _lib.current_stream(self.device)), "ix_arena_create")
        if rc != _lib.IX_OK:
            raise RuntimeError("[isoexec-gdn] this device does not support virtual-memory arenas; unset "
                               f"{_CPR_SLEEP_ENV}")
        self._handle = handle
        self.base = int(_lib.lib().ix_arena_base(handle))
        self.nbytes = int(_lib.lib().ix_arena_bytes(handle))

    @property
    def mapped(self) -> bool:
        return bool(_lib.lib().ix_arena_is_mapped(self._handle))

    @property
    def __cuda_array_interface__(self):
        return {"shape": (self.nbytes,), "typestr": "|u1", "data": (self.base, False), "version": 2}

    def tensor(self) -> torch.Tensor:
        """The arena's bytes as a tensor (no copy). Valid only while the memory is mapped."""
        if not self.mapped:
            raise RuntimeError("[isoexec-gdn] the arena's memory is released")
        return torch.as_tensor(self, device=self.device)

    def release_memory(self) -> None:
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().ix_arena_release_memory(self._handle), "ix_arena_release_memory")

    def restore_memory(self) -> None:
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().ix_arena_restore_memory(self._handle, _lib.current_stream(self.device)),
                       "ix_arena_restore_memory")

    def destroy(self) -> None:
        if self._handle is not None:
            with torch.cuda.device(self.device):
                _lib.check(_lib.lib().ix_arena_destroy(self._handle), "ix_arena_destroy")
            self._handle = None


def _carve(specs, device, arena: Optional[DeviceArena] = None, make_arena: bool = False):
    """One zeroed flat allocation (an ordinary one, or a ``DeviceArena``'s bytes) and the views the specs name, each on a
    256-byte boundary. Returns ``(flat, views, arena)``."""
    offsets, at = [], 0
    for _name, shape, dtype in specs:
        offsets.append(at)
        at += (int(np.prod(shape)) * torch.empty((), dtype=dtype).element_size() + 255) // 256 * 256
    if arena is None and make_arena:
        arena = DeviceArena(at, device)
    flat = arena.tensor()[:at] if arena is not None else torch.zeros(at, dtype=torch.uint8, device=device)
    views = {}
    for (name, shape, dtype), off in zip(specs, offsets):
        n = int(np.prod(shape)) * torch.empty((), dtype=dtype).element_size()
        views[name] = flat[off:off + n].view(dtype).view(shape)
    return flat, views, arena


def cpr_arena_bytes(layers=None) -> int:
    return sum(ly._flat_arena.numel() for ly in (CPR_LAYERS if layers is None else layers) if ly._flat_arena is not None)


def cpr_sleep(layers=None, *, empty_cache: bool = True) -> int:
    """Give every layer's state back to the device (no host copy: the state of a sleeping engine is not kept) after
    dropping the boundary store. Returns the bytes released."""
    layers = list(CPR_LAYERS if layers is None else layers)
    cpr_apc_store_invalidate()
    released = sum(ly._release_arena() for ly in layers)
    if empty_cache and released and torch.cuda.is_available():
        torch.cuda.empty_cache()
    return released


def cpr_wake(layers=None) -> int:
    """Make the state of every sleeping layer anew: zeroed, every row released. Returns the bytes allocated."""
    return sum(ly._restore_arena() for ly in (CPR_LAYERS if layers is None else layers))


def build_cpr_gdn(*, max_num_seqs: int, chunk_size: int, **kw) -> "CprGDN":
    """gdn_cpr_state.py:374-376."""
    return CprGDN(capacity=max_num_seqs, chunk_size=chunk_size, **kw)


class CprGDN(RecurrentGDN):
    """RecurrentGDN + per-row open-chunk buffers, fp32 entry states and the boundary pass."""

    def __init__(self, *, capacity: int, chunk_size: int, ssm_state=None, conv_state=None, **kw):
        if ssm_state is not None or conv_state is not None:
            raise ValueError("[isoexec-gdn] cpr mode owns its state pool (entry states and open-chunk buffers live "
                             "beside it); engine-owned state tensors are not supported.")
        if chunk_size < 2:
            raise ValueError("chunk_size must be at least 2")
        super().__init__(capacity=capacity, **kw)
        rows = capacity + 1
        C = int(chunk_size)
        HV, K, V, H = self.num_v_heads, self.head_k_dim, self.head_v_dim, self.num_k_heads
        dev, dt = self.ssm_state.device, self.conv_state.dtype
        self.chunk_size = C
        # the running and convolution states, the fp32 entry states and the open-chunk buffers (prepared values, as
        # the boundary pass consumes them: k normalised, g fp32, beta in the wire dtype) are views into one allocation
        self._arena_specs = cpr_arena_specs(rows=rows, C=C, HV=HV, K=K, V=V, Hk=H, dt=dt, gdt=torch.float32,
                                            conv_shape=self.conv_state.shape)
        self._arena_device = dev
        self._flat_arena = None
        self._device_arena = None              # a DeviceArena when the state keeps its address over a sleep
        self._stable_address = cpr_sleep_enabled()
        self._restore_arena(release_rows=False)
        # row -> [(boundary position, fp32 entry state, convolution window)] stashed by the last prefill
        self._apc = cpr_apc_enabled()
        self._apc_pending: dict = {}
        # absolute position (tokens consumed) per row; pos % C is how full the open chunk is
        self.pos = torch.zeros(rows, dtype=torch.int64, device=dev)
        # rows whose boundary pass is pending inside the current decode step (row id, or 0)
        self._due = torch.zeros(rows, dtype=torch.int32, device=dev)
        self._cu_pool = torch.arange(0, (rows + 1) * C, C, dtype=torch.int32, device=dev)
        CPR_LAYERS.append(self)

    # -- sleep
    @property
    def asleep(self) -> bool:
        return self._flat_arena is None

    def _release_arena(self) -> int:
        if self._flat_arena is None:
            return 0
        size = self._flat_arena.numel()
        self._flat_arena = None
        for name, _shape, _dtype in self._arena_specs:
            setattr(self, name, None)
        self._apc_pending.clear()
        if self._device_arena is not None:
            self._device_arena.release_memory()  # synchronises the device first
        return size

    def _restore_arena(self, release_rows: bool = True) -> int:
        if self._flat_arena is not None:
            return 0
        if self._device_arena is not None:
            self._device_arena.restore_memory()  # the same addresses, fresh zeroed memory
        self._flat_arena, views, self._device_arena = _carve(self._arena_specs, self._arena_device, self._device_arena,
                                                             make_arena=self._stable_address)
        for name, view in views.items():
            setattr(self, name, view)
        if release_rows:  # what the rows held is gone: nobody may resume from them
            self.table.release_all()
            self.flush_slot_map()
            self.last_used.zero_()
            self._clock.zero_()
            self.pos.zero_()
            self._due.zero_()
        return self._flat_arena.numel()

    def _awake(self) -> None:
        if self._flat_arena is None:
            raise RuntimeError("[isoexec-gdn] this layer's state was released by cpr_sleep; call cpr_wake first")

    # -- row lifecycle
    def _reset_rows(self, rows) -> None:
        if len(rows) == 0:
            return
        t = torch.tensor(list(rows), dtype=torch.long, device=self.pos.device)
        self.pos[t] = 0
        if self.entry_state is not None:
            self.entry_state[t] = 0.0
        for r in rows:
            self._apc_pending.pop(int(r), None)

    def _on_row_released(self, row: int) -> None:
        self._reset_rows([row])

    def _zero_fresh_rows(self, fresh_rows: torch.Tensor) -> None:
        super()._zero_fresh_rows(fresh_rows)
        self.entry_state.index_fill_(0, fresh_rows, 0.0)
        self.pos.index_fill_(0, fresh_rows, 0)
        self.pos[0] = 0  # "none" is spelled row 0

    def reset(self) -> int:
        self._awake()
        freed = super().reset()
        self.entry_state.zero_()
        self.pos.zero_()
        self._due.zero_()
        self._apc_pending.clear()
        return freed

    # -- boundary checkpoints of a prefill call
    def _apc_capture(self, x, rows, qsl, pos0, lens, nb, snaps) -> None:
        """Stash ``(position, fp32 entry state, convolution window)`` for the last two boundaries each sequence closed
        in this call. A boundary is taken only when its whole window of W-1 inputs lies inside this call's ``x``;
        one that does not is skipped, never pieced together (gdn_cpr_state.py:555-578)."""
        W = self.conv_weight.shape[-1]
        C = self.chunk_size
        for i, m in enumerate(nb):
            if not m:
                continue
            if len(self._apc_pending) >= _APC_PENDING_MAX:
                break
            first = (pos0[i] // C + 1) * C            # the first boundary this call closed
            stash = []
            for j in range(max(0, m - 2), m):
                at = first + j * C
                inside = at - pos0[i]                    # tokens of this call in front of the boundary
                if inside < W - 1 or inside > lens[i]:
                    continue
                t = int(qsl[i]) + inside                 # row of x of the token after the boundary
                stash.append((at, snaps[i][j].detach().clone(), x[t - (W - 1):t].transpose(0, 1).contiguous()))
            if stash:
                self._apc_pending[rows[i]] = stash

    # -- the boundary pass of a decode step (host-free)
    def _boundary_pass(self) -> None:
        """State-only scan of every due row's C buffered tokens from its entry state, then the hand-off to the
        running state. Rows that are not due are null lanes of the scan."""
        C, rows = self.chunk_size, self.pos.numel()
        flat = lambda t: t.view(1, rows * C, *t.shape[2:])
        gdn_recurrent_kernel(flat(self.k_buf), flat(self.k_buf), flat(self.v_buf), flat(self.g_buf), flat(self.b_buf),
                             ssm_state=self.entry_state, state_indices=self._due, cu_seqlens=self._cu_pool,
                             want_output=False)
        elems = self.entry_state[0].numel()
        _lib.check(
            _lib.lib().ix_gdn_cpr_handoff(self.entry_state.data_ptr(), self.ssm_state.data_ptr(), self._due.data_ptr(),
                                          rows, elems, _lib.dtype_code(self.k_buf.dtype),
                                          _lib.current_stream(self.pos.device)), "ix_gdn_cpr_handoff")

    @torch.no_grad()
    def decode(self, slots: torch.Tensor, x: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """One decode step for N requests, the buffer append, and the boundary pass where a chunk closed."""
        from .gdn_ops import conv_packed

        self._awake()
        N = x.shape[0]
        rows32 = self._decode_rows(slots)
        cu = self._decode_cu.get(N)
        if cu is None:
            cu = self._decode_cu[N] = torch.arange(N + 1, dtype=torch.int32, device=x.device)
        q, k, v, g, beta = self._decode_prepare(x, a, b, rows32, cu)
        o = gdn_recurrent_kernel(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), g.unsqueeze(0), beta.unsqueeze(0),
                                 ssm_state=self.ssm_state, state_indices=rows32, cu_seqlens=cu, time_tile=1)
        H, K, HV, V = self.num_k_heads, self.head_k_dim, self.num_v_heads, self.head_v_dim
        _lib.check(
            _lib.lib().ix_gdn_cpr_scatter(k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), g.data_ptr(),
                                          beta.data_ptr(), rows32.data_ptr(), self.pos.data_ptr(),
                                          self.k_buf.data_ptr(), self.v_buf.data_ptr(), self.g_buf.data_ptr(),
                                          self.b_buf.data_ptr(), self._due.data_ptr(), _lib.dtype_code(k.dtype), N, H, K,
                                          HV, V, self.chunk_size, _lib.current_stream(x.device)), "ix_gdn_cpr_scatter")
        self._boundary_pass()
        return o[0]

    @torch.no_grad()
    def prefill(self, slots, slots_cpu, x, a, b, qsl, has_initial_state=None, prefill_query_start_loc=None,
                fuse_l2norm: bool = True):
        """Prefill a packed batch of N prompts or prompt chunks (a resumed row continues at its stored position,
        which may be inside an open chunk). Returns ``o [T, HV, V]``. ``fuse_l2norm=False`` keeps the convolution and
        the l2norm apart (a traced run: each op's output is a region of its own); the same bits."""
        self._awake()
        rows, is_cont, _rows_out, cu, q, k, v, g, beta = self._prefill_prepare(
            slots_cpu, x, a, b, qsl, has_initial_state, prefill_query_start_loc, fuse_l2norm=fuse_l2norm)
        C = self.chunk_size
        dev = x.device
        N = len(rows)
        lens = [int(qsl[i + 1] - qsl[i]) for i in range(N)]
        rows_t = torch.tensor(rows, dtype=torch.long, device=dev)
        pos_dev = self.pos[rows_t].tolist() if any(is_cont) else [0] * N
        pos0 = [p if c else 0 for p, c in zip(pos_dev, is_cont)]
        H, K, HV, V = self.num_k_heads, self.head_k_dim, self.num_v_heads, self.head_v_dim

        # ---- the chain: entry states at every boundary crossed by this call
        nb = [(p + n) // C - p // C for p, n in zip(pos0, lens)]
        snaps = [None] * N  # per sequence: fp32 boundary states [nb, HV, V, K] (the last one is the new entry)
        if any(nb):
            ck, cv, cg, cb, clens = [], [], [], [], []
            for i, (p, n, m) in enumerate(zip(pos0, lens, nb)):
                if m == 0:
                    clens.append(0)
                    continue
                r0 = p % C
                take = m * C - r0  # new tokens up to the last boundary crossed
                t0 = int(qsl[i])
                ck += [self.k_buf[rows[i], :r0], k[t0:t0 + take]]
                cv += [self.v_buf[rows[i], :r0], v[t0:t0 + take]]
                cg += [self.g_buf[rows[i], :r0], g[t0:t0 + take]]
                cb += [self.b_buf[rows[i], :r0], beta[t0:t0 + take]]
                clens.append(m * C)
            ccu = torch.tensor(np.concatenate([[0], np.cumsum(clens)]), dtype=torch.int32, device=dev)
            h, final, _ = chunk_boundary_states(
                None, torch.cat(ck).unsqueeze(0), torch.cat(cv).unsqueeze(0), torch.cat(cg).unsqueeze(0),
                torch.cat(cb).unsqueeze(0), ccu, C, initial_state=self.entry_state[rows_t], output_final_state=True,
                lens=clens, keep_fp32=True)
            at = 0
            for i, m in enumerate(nb):
                if m:
                    # h[at] is the state entering the chain's first chunk (the old entry); boundaries 1..m-1 follow
                    snaps[i] = torch.cat([h[0, at + 1:at + m], final[i:i + 1]], 0)
                    at += m
            crossed = [i for i, m in enumerate(nb) if m]
            ct = torch.tensor([rows[i] for i in crossed], dtype=torch.long, device=dev)
            self.entry_state[ct] = torch.stack([snaps[i][-1] for i in crossed])
            if self._apc:
                self._apc_capture(x, rows, qsl, pos0, lens, nb, snaps)

        # ---- the outputs: one segmented scan of the new tokens
        wire = k.dtype
        seg_off, seg_src = [0], []  # per segment: ("run", i) = from the running state of sequence i, or a snapshot
        last_seg = [None] * N
        for i, (p, n) in enumerate(zip(pos0, lens)):
            done, j = 0, 0
            while done < n:
                room = C - (p + done) % C
                take = min(room, n - done)
                seg_src.append(("run", i) if done == 0 else ("snap", i, j - 1))
                last_seg[i] = len(seg_src) - 1
                seg_off.append(seg_off[-1] + take)
                done += take
                j += 1
        M = len(seg_src)
        out = torch.empty(x.shape[0], HV, V, dtype=wire, device=dev)
        if M:
            pool = torch.empty(M + 1, HV, V, K, dtype=torch.float32, device=dev)
            pool[0].zero_()
            run_rows = [s for s, src in enumerate(seg_src) if src[0] == "run"]
            pool[torch.tensor([s + 1 for s in run_rows], dtype=torch.long, device=dev)] = \
                self.ssm_state[torch.tensor([rows[seg_src[s][1]] for s in run_rows], dtype=torch.long, device=dev)]
            for s, src in enumerate(seg_src):
                if src[0] == "snap":
                    pool[s + 1] = snaps[src[1]][src[2]].to(wire).to(torch.float32)
            idx = np.zeros((M, C), dtype=np.int32)
            seg_len = np.diff(seg_off)
            idx[:, 0] = np.arange(1, M + 1)
            for i in range(N):
                if last_seg[i] is not None:
                    s = last_seg[i]
                    idx[s, seg_len[s] - 1] = s + 1  # the running state after the sequence's last token
            # the packed new tokens in segment order ARE the packed batch: segments only cut sequences
            o = gdn_recurrent_kernel(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), g.unsqueeze(0), beta.unsqueeze(0),
                                     ssm_state=pool, state_indices=torch.from_numpy(idx).to(dev),
                                     cu_seqlens=torch.tensor(seg_off, dtype=torch.int32, device=dev))
            out = o[0]
            live = [i for i in range(N) if last_seg[i] is not None]
            lt = torch.tensor([rows[i] for i in live], dtype=torch.long, device=dev)
            self.ssm_state[lt] = pool[torch.tensor([last_seg[i] + 1 for i in live], dtype=torch.long, device=dev)]

        # ---- open-chunk buffers, positions, and the hand-off for rows that end exactly on a boundary
        for i, (p, n, m) in enumerate(zip(pos0, lens, nb)):
            if n == 0:
                continue
            end = p + n
            tail = end % C
            t1 = int(qsl[i + 1])
            lo = (p % C) if m == 0 else 0
            cnt = tail - lo
            if cnt > 0:
                sl = slice(t1 - cnt, t1)
                self.k_buf[rows[i], lo:tail] = k[sl]
                self.v_buf[rows[i], lo:tail] = v[sl]
                self.g_buf[rows[i], lo:tail] = g[sl]
                self.b_buf[rows[i], lo:tail] = beta[sl]
            if tail == 0 and m:
                self.ssm_state[rows[i]] = snaps[i][-1].to(wire).to(torch.float32)
        self.pos[rows_t] = torch.tensor([p + n for p, n in zip(pos0, lens)], dtype=torch.int64, device=dev)
        self.pos[0] = 0
        return out
