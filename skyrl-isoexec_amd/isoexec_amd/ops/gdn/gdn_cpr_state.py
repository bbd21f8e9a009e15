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

Not carried over from the reference: its sleep arenas and prefix-cache store (engine plumbing around the same state).
"""
from __future__ import annotations

import numpy as np
import torch

from ... import _lib
from .gdn_cpr import chunk_boundary_states
from .gdn_ops import gdn_recurrent_kernel
from .gdn_recurrent_state import RecurrentGDN

CPR_LAYERS: list = []


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
        self.entry_state = torch.zeros(rows, HV, V, K, dtype=torch.float32, device=dev)
        # prepared values, as the boundary pass consumes them (k normalised, g fp32, beta in the wire dtype)
        self.k_buf = torch.zeros(rows, C, H, K, dtype=dt, device=dev)
        self.v_buf = torch.zeros(rows, C, HV, V, dtype=dt, device=dev)
        self.g_buf = torch.zeros(rows, C, HV, dtype=torch.float32, device=dev)
        self.b_buf = torch.zeros(rows, C, HV, dtype=dt, device=dev)
        # absolute position (tokens consumed) per row; pos % C is how full the open chunk is
        self.pos = torch.zeros(rows, dtype=torch.int64, device=dev)
        # rows whose boundary pass is pending inside the current decode step (row id, or 0)
        self._due = torch.zeros(rows, dtype=torch.int32, device=dev)
        self._cu_pool = torch.arange(0, (rows + 1) * C, C, dtype=torch.int32, device=dev)
        CPR_LAYERS.append(self)

    # -- row lifecycle
    def _reset_rows(self, rows) -> None:
        if len(rows) == 0:
            return
        t = torch.tensor(list(rows), dtype=torch.long, device=self.pos.device)
        self.pos[t] = 0
        self.entry_state[t] = 0.0

    def _on_row_released(self, row: int) -> None:
        self._reset_rows([row])

    def _zero_fresh_rows(self, fresh_rows: torch.Tensor) -> None:
        super()._zero_fresh_rows(fresh_rows)
        self.entry_state.index_fill_(0, fresh_rows, 0.0)
        self.pos.index_fill_(0, fresh_rows, 0)
        self.pos[0] = 0  # "none" is spelled row 0

    def reset(self) -> int:
        freed = super().reset()
        self.entry_state.zero_()
        self.pos.zero_()
        self._due.zero_()
        return freed

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
    def prefill(self, slots, slots_cpu, x, a, b, qsl, has_initial_state=None, prefill_query_start_loc=None):
        """Prefill a packed batch of N prompts or prompt chunks (a resumed row continues at its stored position,
        which may be inside an open chunk). Returns ``o [T, HV, V]``."""
        rows, is_cont, _rows_out, cu, q, k, v, g, beta = self._prefill_prepare(
            slots_cpu, x, a, b, qsl, has_initial_state, prefill_query_start_loc)
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
