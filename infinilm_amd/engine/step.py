"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

A step runs only the tokens it is given, as one flattened batch, from the cache that earlier steps
left: portions of prompts beside single decoded tokens, cut anywhere.  Reference for the tensors a
step carries: python/infinilm/processors/basic_llm_processor.py:161-263 (token ids, positions,
lengths, offsets, block tables padded with -1, slot mapping) and csrc/engine/infer_engine.cpp:187-254
(copy to the device once per step).  Unlike the reference, positions are derived from the cache
manager's record of each request, all metadata goes to the device in one copy, and there is one
attention contract for every kind of segment (the reference switches kernels by `T != R`,
csrc/layers/attention/backends/paged_attn.cpp:36-37).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import kernels
from ..cache import CacheError, CacheManager


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""
    req_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # for models whose positions have several axes (`ModelSpec.position_axes`): [axes][len(tokens)] positions for
    # the encoding; None: every axis is the token's place in its sequence
    positions: Optional[Sequence[Sequence[int]]] = None


class StepBatch:
    """Device-side metadata of one step (all int32), plus a few host-side facts kernels dispatch on."""

    def __init__(self):
        self.T = 0                      # tokens in the step
        self.R = 0                      # requests in the step
        self.token_ids = None           # [T]
        self.positions = None           # [T] absolute position of each token in its request (what the cache and the attention count by)
        self.position_axes = None       # [axes, T] positions for the encoding; with one axis, the same numbers
        self.seg_of_token = None        # [T] index of the token's request in this batch
        self.seg_offsets = None         # [R+1] prefix sums of new-token counts
        self.start_pos = None           # [R] tokens cached before this step
        self.total_lens = None          # [R] tokens cached after this step
        self.want_rows = None           # [num_wanted] rows of the flattened batch
        self.state_in = None            # [R] state row read at the start (0 = zeros)
        self.state_out = None           # [R] state row written at the end
        self.att_tiles = None           # [n, 2] (first row, count): runs of <= 8 consecutive tokens of one request
        self.att_single_rows = None     # rows of requests that bring one token (None: no run of 2 or more exists)
        self.block_tables: List = []    # per group [R, max_blocks], -1 padded
        self.slots: List = []           # per group [T] slot of each new token
        self.num_wanted = 0
        self.wants_all_rows = False
        self.max_q_len = 0
        self.max_total_len = 0
        self.max_position = 0
        self.all_decode = False
        # host copies for parts that plan on the host
        self.h_seg_offsets: Optional[np.ndarray] = None
        self.h_start_pos: Optional[np.ndarray] = None
        self.h_state_in: Optional[np.ndarray] = None
        self.h_state_out: Optional[np.ndarray] = None
        self.taps: Optional[dict] = None


class StepRunner:
    """Owns the model and the cache manager; `step()` is the one function that advances requests."""

    def __init__(self, model, cache: CacheManager, enable_graph: bool = False):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.enable_graph = bool(enable_graph)
        self._graphs: Dict = {}          # (requests, block-table width) -> (graph, batch, logits, buffer)
        self._graph_pool = None
        self._graph_seen: Dict = {}      # sizes met in eager steps so far -> how often
        self.graph_after = 2
        # steps with portions of prompts are recorded too, by their bounded shape, where every layer's parts say that they
        # take their indices from the device's tensors in such steps
        self.graph_mixed = all(getattr(b, "records_mixed_steps", False) for b in getattr(model, "blocks", []))
        self.graph_mixed_max_tokens = 8192   # ... up to this many tokens a step (a recording keeps the step's activations)
        self.graph_mixed_pad_share = 8       # ... whose bounded shape adds at most 1/8 of rows of no request (0: any)
        self._pinned: List[Optional[torch.Tensor]] = [None, None]   # two staging buffers in turn
        self._copy_done: List[Optional[torch.cuda.Event]] = [None, None]
        self._stage_turn = 0
        self._prepared = None            # metadata of the next decode step, built while the device ran this one
        self.steps = 0
        self.tokens = 0

    # ---- batch building -----------------------------------------------------------------------
    def _stage(self, n: int) -> torch.Tensor:
        """Pinned host memory for a step's metadata; two buffers in turn, each waited for only when its
        own last copy to the device may still be reading it."""
        t = self._stage_turn = self._stage_turn ^ 1
        if self._copy_done[t] is not None:
            self._copy_done[t].synchronize()
            self._copy_done[t] = None
        if self._pinned[t] is None or self._pinned[t].numel() < n:
            self._pinned[t] = torch.empty((max(n, 4096) * 2,), dtype=torch.int32, pin_memory=self.device.type == "cuda")
        return self._pinned[t][:n]

    def _copy_to_device(self, dev: torch.Tensor, host: torch.Tensor, turn: int) -> None:
        dev.copy_(host, non_blocking=True)
        if self.device.type == "cuda":
            self._copy_done[turn] = torch.cuda.Event()
            self._copy_done[turn].record()

    def build_batch(self, entries: Sequence[StepEntry], min_blocks: int = 0,
                    device_buffer: Optional[torch.Tensor] = None, defer_copy: bool = False,
                    pad_rows: int = 0, bounds: Optional[tuple] = None) -> StepBatch:
        """Reserves pages for every entry and lays the step's metadata out.

        `min_blocks` pads the block tables to a fixed width and `device_buffer` receives the
        metadata instead of a fresh tensor: a captured graph reads the same addresses at every
        replay.  `defer_copy`: the metadata stays in its staging buffer (`batch.pending_copy`): the
        caller fills in the token ids and sends it later.  `pad_rows` (steps of single tokens only):
        that many rows of no request follow the entries' rows, so that one recorded step serves every
        number of requests up to its size: each is a token 0 at position 0 of a sequence of one token
        whose only page is the cache's page for such rows; its logits are computed and not returned.
        Such rows write their key and value to slot (row number mod page size) of that page: with more of
        them than the page holds, several write the same slot in one launch, and all of them read key 0
        of the page, which the first of them rewrites every step.  Harmless, because nothing of such a row
        is ever returned and the page belongs to no request; no other page is touched.
        `bounds` = (requests, wanted rows, attention tiles, single rows): every array of the metadata is laid out
        for that many entries (with `pad_rows` and `min_blocks` for the tokens and the block tables), so that a
        recorded step of mixed content finds every array at the same address at every replay: lists are
        filled up with entries that do nothing (tiles of no tokens, a single row or a wanted row once more)."""
        cache = self.cache
        V = self.model.spec.vocab_size
        if not entries and not pad_rows:
            raise ValueError("a step needs at least one entry")
        if not entries:
            min_blocks = max(min_blocks, 1)
        if not defer_copy:
            # prepared metadata lies in one of the two staging buffers that this step and the next take
            # in turn: it does not outlive a step built in between
            self._prepared = None
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            n = len(e.tokens)
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
            for t in e.tokens:
                if not 0 <= t < V:
                    raise ValueError(f"request {e.req_id!r}: token id {t} is outside the vocabulary of {V}")
            if e.positions is not None and (len(e.positions) != self.model.spec.position_axes
                                            or any(len(ax) != n for ax in e.positions)):
                raise ValueError(f"request {e.req_id!r}: positions must be [{self.model.spec.position_axes}][{n}]")
            if cache.length(e.req_id) + n > self.model.spec.max_positions:
                raise ValueError(f"request {e.req_id!r}: {cache.length(e.req_id) + n} tokens exceed the model's "
                                 f"{self.model.spec.max_positions} positions")
        reserved = []
        try:
            for e in entries:
                cache.reserve(e.req_id, len(e.tokens))
                reserved.append(e)
        except Exception:
            # pages taken for earlier entries of this step stay with their requests (they will be
            # used by the same tokens later); nothing is half-written
            raise

        R_real = len(entries)
        if pad_rows and bounds is None and any(len(e.tokens) != 1 for e in entries):
            raise ValueError("rows of no request fill up steps of single tokens only")
        # rows of no request: a sequence of one token each after decoded tokens; after a mixed step's tokens
        # (bounded layout) one segment that holds them all, every one at position 0
        pad_segs = int(pad_rows) if bounds is None else (1 if pad_rows else 0)
        R = R_real + pad_segs
        lens = np.ones(R, dtype=np.int64)
        lens[:R_real] = [len(e.tokens) for e in entries]
        if bounds is not None and pad_rows:
            lens[R_real] = int(pad_rows)
        T = int(lens.sum())
        start = np.zeros(R, dtype=np.int64)
        start[:R_real] = [cache.length(e.req_id) for e in entries]
        offsets = np.zeros(R + 1, dtype=np.int64)
        np.cumsum(lens, out=offsets[1:])
        G = len(cache.groups)
        ps = cache.page_size
        max_blocks = [max(1, min_blocks, max((len(cache.table(e.req_id, g)) for e in entries), default=0)) for g in range(G)]
        n_want = sum(len(e.want) for e in entries) + (int(pad_rows) if bounds is None else 0)

        # attention work lists: runs of up to TILE consecutive tokens of a request, and single tokens
        TILE = kernels.ATT_TILE_TOKENS
        tiles: List[int] = []
        singles: List[int] = []
        for i in range(R_real):
            a, n = int(offsets[i]), int(lens[i])
            if n == 1:
                singles.append(a)
            else:
                for k in range(0, n, TILE):
                    tiles += [a + k, min(TILE, n - k)]
        if not tiles and bounds is None:
            singles = []   # every token is single: the kernels take all rows
        # (the rows of no request of a bounded layout are left out of the attention: nothing reads what they hold)
        R_lay, want_lay, tiles_lay, singles_lay = R, n_want, len(tiles) // 2, len(singles)
        if bounds is not None:
            R_lay, want_lay, tiles_lay, singles_lay = bounds
            if R > R_lay or n_want > want_lay or len(tiles) // 2 > tiles_lay or len(singles) > singles_lay:
                raise RuntimeError("a step does not fit the bounds it is laid out for")

        # layout of the one int32 buffer
        axes = int(getattr(self.model.spec, "position_axes", 1))
        sizes = [("token_ids", T), ("positions", T), ("axes", (axes if axes > 1 else 0) * T), ("seg_of_token", T), ("seg_offsets", R_lay + 1), ("start_pos", R_lay),
                 ("total_lens", R_lay), ("want_rows", want_lay), ("state_in", R_lay), ("state_out", R_lay),
                 ("att_tiles", 2 * tiles_lay), ("att_singles", singles_lay)]
        for g in range(G):
            sizes.append((f"slots{g}", T))
            sizes.append((f"bt{g}", R_lay * max_blocks[g]))
        off = {}
        total = 0
        for name, n in sizes:
            off[name] = (total, n)
            total += (n + 3) // 4 * 4  # keep every array 16-byte aligned
        host = self._stage(total)
        h = host.numpy()

        def seg(name):
            o, n = off[name]
            return h[o:o + n]

        seg("token_ids")[:T - pad_rows] = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=T - pad_rows)
        seg("token_ids")[T - pad_rows:] = 0
        pos = seg("positions")
        sot = seg("seg_of_token")
        all_single = T == R
        if all_single:   # decoded tokens only: no per-entry array work
            pos[:] = start
            sot[:] = np.arange(R)
        else:
            for i in range(R):
                a, b = offsets[i], offsets[i + 1]
                pos[a:b] = np.arange(start[i], start[i] + lens[i]) if i < R_real else 0
                sot[a:b] = i
        if axes > 1:   # every axis the place in the sequence, unless the entry brings its own
            ax = seg("axes").reshape(axes, T)
            ax[:] = pos[None, :]
            for i, e in enumerate(entries):
                if e.positions is not None:
                    ax[:, offsets[i]:offsets[i + 1]] = np.asarray(e.positions, dtype=np.int64)
        seg("seg_offsets")[:R + 1] = offsets
        seg("seg_offsets")[R + 1:] = T
        seg("start_pos")[:R] = start
        seg("start_pos")[R:] = 0
        seg("total_lens")[:R] = start + lens
        seg("total_lens")[R_real:] = 1
        w = seg("want_rows")
        k = 0
        for i, e in enumerate(entries):
            for x in e.want:
                w[k] = offsets[i] + x
                k += 1
        if bounds is None:
            for i in range(R_real, R):
                w[k] = offsets[i]
                k += 1
        w[k:] = w[k - 1] if k else T - 1   # (a bounded layout: the last wanted row once more)
        at = seg("att_tiles")
        at[:len(tiles)] = tiles
        at[len(tiles):] = 0             # tiles of no tokens
        asg = seg("att_singles")
        asg[:len(singles)] = singles
        asg[len(singles):] = -1         # no row: the kernels skip such entries
        sin, sout = seg("state_in"), seg("state_out")
        for i, e in enumerate(entries):
            sin[i], sout[i] = cache.state_rows(e.req_id)
        sin[R_real:] = 0
        sout[R_real:] = cache.null_state_row
        for g in range(G):
            sl = seg(f"slots{g}")
            bt = seg(f"bt{g}").reshape(R_lay, max_blocks[g])
            bt[:] = -1
            if all_single:
                slot_list = []
                bt[R_real:, 0] = cache.null_page(g)
                for i, e in enumerate(entries):
                    table = cache.table(e.req_id, g)
                    bt[i, :len(table)] = table
                    p = int(start[i])
                    page = table[p // ps]
                    if page < 0:
                        raise RuntimeError(f"request {e.req_id!r}: a new token falls on a page already given back")
                    slot_list.append(page * ps + p % ps)
                slot_list += [cache.null_page(g) * ps + i % ps for i in range(pad_rows)]
                sl[:] = slot_list
                continue
            for i, e in enumerate(entries):
                table = np.asarray(cache.table(e.req_id, g), dtype=np.int64)
                bt[i, :len(table)] = table
                p = np.arange(start[i], start[i] + lens[i])
                pages = table[p // ps]
                if (pages < 0).any():
                    raise RuntimeError(f"request {e.req_id!r}: a new token falls on a page already given back")
                sl[offsets[i]:offsets[i + 1]] = pages * ps + p % ps
            if pad_rows:   # rows of no request after a mixed step's tokens
                bt[R_real:R, 0] = cache.null_page(g)
                sl[offsets[R_real]:] = cache.null_page(g) * ps + np.arange(pad_rows) % ps

        if device_buffer is None:
            dev = torch.empty((total,), dtype=torch.int32, device=self.device)
        else:
            if device_buffer.numel() < total:
                raise RuntimeError("the graph's metadata buffer is too small for this step")
            dev = device_buffer[:total]
        if not defer_copy:
            self._copy_to_device(dev, host, self._stage_turn)

        def dseg(name):
            o, n = off[name]
            return dev[o:o + n]

        b = StepBatch()
        b.T, b.R = T, R
        b.token_ids, b.positions, b.seg_of_token = dseg("token_ids"), dseg("positions"), dseg("seg_of_token")
        b.position_axes = dseg("axes").view(axes, T) if axes > 1 else b.positions.view(1, T)
        b.seg_offsets, b.start_pos, b.total_lens = dseg("seg_offsets"), dseg("start_pos"), dseg("total_lens")
        b.want_rows, b.state_in, b.state_out = dseg("want_rows"), dseg("state_in"), dseg("state_out")
        b.layout_size = total
        if tiles or bounds is not None:
            b.att_tiles = dseg("att_tiles").view(-1, 2)
            b.att_single_rows = dseg("att_singles") if singles_lay else None
        b.block_tables = [dseg(f"bt{g}").view(R_lay, max_blocks[g]) for g in range(G)]
        b.slots = [dseg(f"slots{g}") for g in range(G)]
        b.num_wanted = want_lay
        b.rows_of_requests = T - int(pad_rows)   # the rows after them belong to no request
        b.wants_all_rows = (bounds is None and n_want == T
                            and all(list(e.want) == list(range(len(e.tokens))) for e in entries))
        b.max_q_len = int(lens.max())
        b.max_total_len = int((start + lens).max())
        b.max_position = b.max_total_len - 1
        b.all_decode = bool((lens == 1).all())
        b.h_seg_offsets = offsets
        b.h_start_pos = start
        b.h_state_in = np.array(sin, dtype=np.int64)
        b.h_state_out = np.array(sout, dtype=np.int64)
        if defer_copy:
            b.pending_copy = (dev, host, self._stage_turn, off["token_ids"][0])
        return b

    # ---- the step -----------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], taps: Optional[dict] = None) -> torch.Tensor:
        """Runs the entries' tokens as one batch and returns float32 logits [wanted, vocab] in the
        order of the entries and of each entry's `want`.

        With `enable_graph`, a step of single decoded tokens that wants each token's logits replays
        a captured HIP graph; the returned tensor is then the graph's output buffer, valid until
        the next such step."""
        if self.enable_graph and taps is None and all(len(e.tokens) == 1 and len(e.want) == 1 and e.want[0] == 0 for e in entries):
            key = self._graph_key(entries)
            if key not in self._graphs:
                self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
            if key in self._graphs or self._graph_seen[key] >= self.graph_after:
                return self._graph_step(entries, key)
        elif self.enable_graph and self.graph_mixed and taps is None and any(len(e.tokens) > 1 for e in entries):
            key = self._mixed_key(entries)
            if key is not None:
                if key not in self._graphs:
                    self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
                if key in self._graphs or self._graph_seen[key] >= self.graph_after:
                    return self._mixed_graph_step(entries, key)
        batch = self.build_batch(entries)
        batch.taps = taps
        logits = self.model.forward(batch, self.cache)
        for e in entries:
            self.cache.commit(e.req_id, len(e.tokens), e.tokens)
        self.steps += 1
        self.tokens += batch.T
        return logits

    # ---- decode steps as captured graphs ----------------------------------------------------------
    def _graph_key(self, entries: Sequence[StepEntry]):
        cache = self.cache
        need = max(-(-(cache.length(e.req_id) + 1) // cache.page_size) for e in entries)
        return (kernels.bound_rows(len(entries)), kernels.bound_pages(need))

    def _graph_step(self, entries: Sequence[StepEntry], key) -> torch.Tensor:
        """One graph per (number of rows, block-table width).  Both are rounded up: the rows to
        `kernels.bound_rows` (1, 2, 4, 8, 16, 24, 32, 48, 64, ...: a step of 5 requests runs as one of 8, filled
        up with rows of no request, so that requests that come and go one by one do not make a recording
        each), the width to `kernels.bound_pages` (4, 6, 8, 12, 16, ... pages), so a graph serves every context up to width * page tokens; the kernels' grids are
        sized for that bound and bound their reads by each request's own length.  Between replays
        only the metadata buffer changes (token ids, positions, slots, block tables).  A size is
        recorded the `graph_after`-th time it comes (a recording costs about three steps, which a
        batch size that passes once, while requests trickle in or out, never earns back).
        Reference: csrc/engine/compiler/paged_compiler.cpp:59-260 (one graph per decode batch size,
        inputs copied into captured buffers)."""
        cache = self.cache
        rows, width = key
        R = len(entries)
        slot = self._graphs.get(key)
        if slot is None:
            graph, batch, logits, buf = self._record(key, entries)
        else:
            graph, batch, logits, buf = slot
            ids = tuple(e.req_id for e in entries)
            prep, self._prepared = self._prepared, None
            if prep is not None and prep[0] == (key, ids, cache.version) and prep[1] == [cache.length(i) for i in ids]:
                # built while the device ran the last step: only the token ids are new
                dev, host, turn, tok_off = prep[2]
                V = self.model.spec.vocab_size
                toks = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=R)
                if toks.min() < 0 or toks.max() >= V:
                    bad = next(e for e in entries if not 0 <= e.tokens[0] < V)
                    raise ValueError(f"request {bad.req_id!r}: token id {bad.tokens[0]} is outside the vocabulary of {V}")
                host.numpy()[tok_off:tok_off + R] = toks
                self._copy_to_device(dev, host, turn)
            else:
                fresh = self.build_batch(entries, min_blocks=width, device_buffer=buf, pad_rows=rows - R)
                if fresh.T != batch.T or [t.shape for t in fresh.block_tables] != [t.shape for t in batch.block_tables]:
                    raise RuntimeError("a decode step does not fit the graph captured for its size")
        graph.replay()
        for e in entries:
            cache.commit(e.req_id, 1, e.tokens)
        self.steps += 1
        self.tokens += R
        self._prepare_next_decode(entries)
        return logits[:R]

    # ---- steps with portions of prompts as captured graphs -------------------------------------------
    def _mixed_key(self, entries: Sequence[StepEntry]):
        """The bounded shape of a step that holds portions of prompts (and decoded tokens beside them): tokens, requests,
        wanted rows and block-table width, each rounded up (`kernels.bound_rows`, `kernels.bound_pages`); the lists of
        attention tiles and of single rows are as long as those allow.  Under a token budget the steps of a busy engine have the budget's tokens and differ in
        the rest by little, so few shapes serve them.  None: not recorded (too many tokens, or a token count that its
        bound would fill up by more than an eighth: a prompt of 1,100 tokens alone would run as 1,536 rows)."""
        cache = self.cache
        T = sum(len(e.tokens) for e in entries)
        if T > self.graph_mixed_max_tokens:
            return None
        if self.graph_mixed_pad_share and kernels.bound_rows(T) - T > T // self.graph_mixed_pad_share:
            return None   # the rows that fill the shape up are computed too: more than an eighth of them is not worth a replay
        n_want = sum(len(e.want) for e in entries)
        need = max(-(-(cache.length(e.req_id) + len(e.tokens)) // cache.page_size) for e in entries)
        return self._mixed_shape(kernels.bound_rows(T), n_want, any(len(e.tokens) == 1 for e in entries), need)

    def _mixed_shape(self, T_b: int, n_want: int, singles: bool, pages: int):
        """The key of a bounded shape.  Requests: as many as the cache takes, and one segment for the rows of no request
        (the lists they size are small; a bound that followed the step's own number would multiply the shapes).  Wanted
        rows: one a request, more if the step asks for more.  Tiles: at most one every TILE tokens and one more a request.
        Single rows: one a request, or none.  Block-table width: a power of two."""
        R_b = kernels.bound_rows(self.cache.max_requests + 1)
        width = 4
        while width < pages:
            width *= 2
        return ("mixed", T_b, R_b, max(R_b, kernels.bound_rows(max(n_want, 1))), T_b // kernels.ATT_TILE_TOKENS + R_b,
                R_b if singles else 0, width)

    def _mixed_graph_step(self, entries: Sequence[StepEntry], key) -> torch.Tensor:
        """Replays (or first records) the step of bounded shape `key` with the entries' tokens first and rows of no
        request after them; only the metadata buffer changes between replays."""
        _, T_b, R_b, want_b, tiles_b, singles_b, width = key
        T = sum(len(e.tokens) for e in entries)
        n_want = sum(len(e.want) for e in entries)
        if len(entries) + 1 > R_b:
            raise RuntimeError("more requests in a step than the cache takes")
        self._prepared = None
        slot = self._graphs.get(key)
        build = lambda buf: self.build_batch(entries, min_blocks=width, device_buffer=buf, pad_rows=T_b - T,
                                             bounds=(R_b, want_b, tiles_b, singles_b))
        if slot is None:
            probe = self.build_batch(entries, min_blocks=width, pad_rows=T_b - T, bounds=(R_b, want_b, tiles_b, singles_b),
                                     defer_copy=True)   # (pages are reserved here; the layout's size is what is wanted)
            buf = torch.zeros((probe.layout_size + 64,), dtype=torch.int32, device=self.device)
            batch = build(buf)
            batch.max_total_len = width * self.cache.page_size
            saved = self.cache.snapshot_states([e.req_id for e in entries])
            self.model.forward(batch, self.cache)      # warm-up outside the capture; the replay writes the same keys again
            self.cache.restore_states(saved)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                logits = self.model.forward(batch, self.cache)
            self._graphs[key] = (graph, batch, logits, buf)
        else:
            graph, batch, logits, buf = slot
            fresh = build(buf)
            if fresh.T != batch.T or fresh.layout_size != batch.layout_size:
                raise RuntimeError("a step does not fit the graph captured for its shape")
        if not entries:
            return logits[:0]    # a recording made ahead of the requests
        graph.replay()
        for e in entries:
            self.cache.commit(e.req_id, len(e.tokens), e.tokens)
        self.steps += 1
        self.tokens += T
        return logits[:n_want]

    def record_mixed_graphs(self, tokens: int, max_context: int) -> int:
        """Records, before any request has come, the steps of `tokens` tokens (a full token budget) with portions of
        prompts, with and without decoded tokens beside them, for every block-table width up to `max_context` tokens:
        returns how many were made."""
        if not (self.enable_graph and self.graph_mixed) or tokens < 2 or tokens > self.graph_mixed_max_tokens:
            return 0
        made = 0
        pages = max(1, -(-int(max_context) // self.cache.page_size)) if self.cache.groups else 1
        widths, w = [], 4
        while True:
            widths.append(w)
            if w >= pages:
                break
            w *= 2
        for width in widths:
            for singles in (True, False):
                key = self._mixed_shape(kernels.bound_rows(tokens), 1, singles, width)
                if key not in self._graphs:
                    self._mixed_graph_step([], key)
                    made += 1
        return made

    def _record(self, key, entries: Sequence[StepEntry]):
        """Records the decode step of size `key` with the entries' rows first and rows of no request
        after them (entries may be empty: a recording made before any request has come)."""
        cache = self.cache
        rows, width = key
        buf = torch.zeros((self._graph_buffer_size(rows, width),), dtype=torch.int32, device=self.device)
        batch = self.build_batch(entries, min_blocks=width, device_buffer=buf, pad_rows=rows - len(entries))
        batch.max_total_len = width * cache.page_size     # grids are sized for the bound, not for this step
        # warm-up outside the capture (libraries set themselves up at their first call).  It runs the
        # step that the first replay runs again: keys and values are written twice with the same
        # values, fixed-size states are put back in between
        saved = cache.snapshot_states([e.req_id for e in entries])
        self.model.forward(batch, cache)
        cache.restore_states(saved)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self.model.forward(batch, cache)
        self._graphs[key] = (graph, batch, logits, buf)
        return self._graphs[key]

    def record_decode_graphs(self, max_rows: int, max_context: int) -> int:
        """Records, before any request has come, the decode steps of every size that up to `max_rows`
        requests with contexts up to `max_context` tokens can need (rows of no request stand in for the
        requests), so that no step of a running service pays for a recording: returns how many were
        made.  The reference records its decode graphs when the engine is built, one a batch size
        (csrc/engine/compiler/paged_compiler.cpp:28-57, :59-260)."""
        if not self.enable_graph or max_rows < 1:
            return 0
        sizes, r = [], 1
        while True:
            sizes.append(kernels.bound_rows(r))
            if sizes[-1] >= max_rows:
                break
            r = sizes[-1] + 1
        pages = max(1, -(-int(max_context) // self.cache.page_size)) if self.cache.groups else 1
        widths, w = [], 1
        while True:
            widths.append(kernels.bound_pages(w))
            if widths[-1] >= pages:
                break
            w = widths[-1] + 1
        made = 0
        for width in widths:
            for rows in sizes:
                if (rows, width) not in self._graphs:
                    self._record((rows, width), [])
                    made += 1
        return made

    def _prepare_next_decode(self, entries: Sequence[StepEntry]) -> None:
        """While the device runs the step just launched: the metadata of the same requests' next decoded
        tokens (positions, slots, block tables; pages reserved), everything but the token ids.  Used by
        the next graph step if it is for these requests at these lengths; else dropped (pages
        reserved here stay with their requests, as after any step that could not run)."""
        cache = self.cache
        try:
            key = self._graph_key(entries)
            slot = self._graphs.get(key)
            if slot is None:
                return
            ids = tuple(e.req_id for e in entries)
            lengths = [cache.length(i) for i in ids]
            if max(lengths) + 1 > self.model.spec.max_positions:
                return
            b = self.build_batch([StepEntry(i, [0], [0]) for i in ids], min_blocks=key[1], device_buffer=slot[3],
                                 defer_copy=True, pad_rows=key[0] - len(ids))
            self._prepared = ((key, ids, cache.version), lengths, b.pending_copy)
        except (CacheError, ValueError):
            self._prepared = None   # out of pages for the guess: the real step will say so if it comes

    # ---- a decode step launched before the tokens of the one before it have come back -------------------
    def ahead_ready(self, ids: Sequence) -> bool:
        """The metadata of these requests' next decoded tokens lies prepared (their pages reserved)
        and a graph for it is recorded: `step_ahead` can launch it without knowing the tokens."""
        prep = self._prepared
        if prep is None or not self.enable_graph:
            return False
        (key, pids, version), lengths, _ = prep
        return (key in self._graphs and pids == tuple(ids) and version == self.cache.version
                and lengths == [self.cache.length(i) for i in pids])

    def step_ahead(self, ids: Sequence, tokens_dev: torch.Tensor) -> torch.Tensor:
        """Launches the decode step whose input tokens are `tokens_dev` (int32 on the device, one a
        request in the order of `ids`: what the sampler of the step before left there) and returns its
        logits buffer.  The host has not seen the tokens: `commit_ahead` completes the step's books
        once it has.  Needs `ahead_ready(ids)`."""
        if not self.ahead_ready(ids):
            raise RuntimeError("no prepared decode step for these requests")
        prep, self._prepared = self._prepared, None
        key = prep[0][0]
        R = len(prep[0][1])
        graph, batch, logits, buf = self._graphs[key]
        dev, host, turn, tok_off = prep[2]
        if tokens_dev.dtype != torch.int32 or tokens_dev.numel() != R or tokens_dev.device != dev.device:
            raise ValueError("the tokens of a step launched ahead are int32 on the device, one a request")
        host.numpy()[tok_off:tok_off + R] = 0
        self._copy_to_device(dev, host, turn)
        dev[tok_off:tok_off + R].copy_(tokens_dev)    # behind the copy above on the stream
        graph.replay()
        self.steps += 1
        self.tokens += R
        return logits[:R]

    def commit_ahead(self, id_tokens: Sequence) -> None:
        """The books of a step launched by `step_ahead`, now that its input tokens are known:
        (request, token) for every request that still exists (one that ended with the step before
        is left out: what the step computed for it is never read).  Then the next step's metadata."""
        live = [(i, t) for i, t in id_tokens if self.cache.has(i)]
        for i, t in live:
            self.cache.commit(i, 1, [t])
        if live:
            self._prepare_next_decode([StepEntry(i, [t], [0]) for i, t in live])

    def _graph_buffer_size(self, R: int, width: int) -> int:
        G = len(self.cache.groups)
        pad = lambda n: (n + 3) // 4 * 4
        axes = int(getattr(self.model.spec, "position_axes", 1))
        return (3 + (axes if axes > 1 else 0)) * pad(R) + pad(R + 1) + 5 * pad(R) + G * (pad(R) + pad(R * width)) + 64
