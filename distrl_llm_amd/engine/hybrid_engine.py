"""Generation engine for layer-list (hybrid) models.

One step function runs a flat batch that mixes portions of prompts with
single decode tokens: every row continues its sequence from the pages and
state slot earlier steps left, however the prompt was cut. ``generate``
is a continuous-batching scheduler over that step (decode tokens first,
prompt portions fill the step's token budget; n-candidate fan-out forks
the prompt's pages and state), with the same call signature as the dense
:class:`Engine`, so the batcher, the server and the command line drive
either. A trace replay (``bin/trace_run``) calls the same step directly.

Numerics: the residual stream, norms, the block's convolution, rotary
angles, attention scores and weights, recurrent state with its decays,
gates and unit norms, router and the residual sum are fp32; matrix
products run in the model dtype with fp32 accumulation (true fp32 when the
model dtype is fp32).
"""

from __future__ import annotations

from typing import List, Optional, Sequence as Seq, Tuple

import torch
import torch.nn.functional as F

from ..config import EngineConfig, SamplingParams
from ..models.hybrid import (DeltaRuleSpec, GluSpec, HybridLM,
                             LatentAttentionSpec, MlpSpec, ParallelMixerSpec,
                             SigmoidAttentionSpec, SinkAttentionSpec,
                             WindowAttentionSpec)
from ..ops import functional as OF
from ..ops import seqmix as SM
from ..utils.capture import collector_paused
from ..utils.trace import trace_range
from .kvcache import Sequence
from .seqstate import LatentCachePool, StateSlotPool


class _DecodeGraph:
    """One captured decode step for a fixed (padded) number of rows.

    All int inputs live in one static device buffer that is refilled by a
    single copy before each replay; rows beyond the live ones point at the
    pools' scratch slot and scratch page, so they compute garbage that
    nothing reads. The state and cache tensors the graph touches are the
    pools' own storages, which live as long as the engine."""

    def __init__(self, eng: "HybridEngine", rows: int):
        self.eng, self.rows = eng, rows
        bs = eng.pool.block_size
        self.max_nb = eng._max_table_width()
        flat, self.lay = self._flat([], [], [], [], [])
        self.host = torch.zeros(len(flat), dtype=torch.int32, pin_memory=True)
        self.host.copy_(torch.tensor(flat, dtype=torch.int32))
        self.buf = self.host.to(eng.device)
        self.copied = torch.cuda.Event()    # the staging buffer's last upload
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):       # lazy initialisation outside the capture
            self._body()
            self._body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with collector_paused(), torch.cuda.graph(self.graph):
            self.logits = self._body()

    def _flat(self, tokens, positions, page_slot, slots, tables):
        eng, n, pad = self.eng, len(tokens), self.rows - len(tokens)
        bs = eng.pool.block_size
        scratch = eng.pool.scratch_block
        meta = dict(positions=positions + [0] * pad,
                    tok_seq=list(range(self.rows)),
                    page_slot=page_slot + [scratch * bs] * pad,
                    cu=list(range(self.rows + 1)),
                    slots=slots + [eng.slots.scratch_slot] * pad,
                    block_tables=tables + [[scratch]] * pad,
                    tiles=[(b, b, 1) for b in range(self.rows)], max_tile=1,
                    wide_tiles=[(b, b, 1) for b in range(self.rows)],
                    max_wide_tile=1)
        return eng._pack(tokens + [0] * pad, meta, list(range(self.rows)),
                         max_nb=self.max_nb)

    def _body(self):
        tok, meta, want = self.eng._views(self.buf, self.lay, 1)
        return self.eng._forward(tok, meta, want)

    def run(self, tokens, meta):
        flat, _ = self._flat(tokens, meta["positions"], meta["page_slot"],
                             meta["slots"], meta["block_tables"])
        self.copied.synchronize()           # do not overwrite an upload in flight
        self.host.copy_(torch.tensor(flat, dtype=torch.int32))
        self.buf.copy_(self.host, non_blocking=True)
        self.copied.record()
        self.graph.replay()
        return self.logits[:len(tokens)]


class HybridEngine:
    def __init__(self, model: HybridLM, cfg: EngineConfig,
                 device: Optional[torch.device] = None, seed: int = 0):
        self.model = model
        self.cfg = cfg
        self.spec = model.spec
        self.device = device if device is not None else model.device
        self.dtype = model.dtype_
        self._seq_counter = 0
        self.generator = torch.Generator(device=self.device)
        self.generator.manual_seed(seed)

        num_slots = cfg.num_state_slots or min(cfg.max_num_seqs, 256)
        num_blocks = cfg.num_kv_blocks
        if num_blocks <= 0:
            num_blocks = self._derive_num_blocks(num_slots)
        self.pool = LatentCachePool(self.spec, num_blocks, cfg.kv_block_size,
                                    self.dtype, self.device)
        self.slots = StateSlotPool(self.spec, num_slots, self.device)
        self._decode_graphs = {}     # padded rows -> _DecodeGraph
        self._consts = {}            # small per-unit device tensors

    def _derive_num_blocks(self, num_slots: int) -> int:
        bs = self.cfg.kv_block_size
        per_block = LatentCachePool.bytes_per_block(self.spec, bs, self.dtype)
        if self.device.type == "cuda":
            free, _ = torch.cuda.mem_get_info(self.device)
            budget = int(free * self.cfg.gpu_memory_utilization)
        else:
            budget = 64 * 1024 * 1024
        n = max(budget // per_block, 16)
        most = num_slots * LatentCachePool.blocks_for(self.cfg.max_seq_length, bs)
        return int(min(n, most))

    # ------------------------------------------------- sequence lifecycle

    def open_sequence(self, prompt_ids: Seq[int] = (), parent_prompt: int = 0
                      ) -> Sequence:
        """Admit a sequence: it gets a zeroed state slot; pages are taken
        as its tokens arrive."""
        self._seq_counter += 1
        q = Sequence(self._seq_counter, list(prompt_ids), parent_prompt)
        q.slot = self.slots.alloc()
        return q

    def close_sequence(self, q: Sequence) -> None:
        """Give a sequence's pages and slot back."""
        q.finished = True
        for b in q.block_table:
            self.pool.allocator.free(b)
        q.block_table = []
        if q.slot is not None:
            self.slots.free(q.slot)
            q.slot = None

    def fork_sequence(self, parent: Sequence) -> Sequence:
        """A new sequence continuing from the parent's state: full pages
        are shared by refcount, a partial last page and the state slot are
        copied."""
        bs = self.pool.block_size
        child = self.open_sequence(parent.prompt_ids, parent.parent_prompt)
        full = parent.context_len // bs
        for b in parent.block_table[:full]:
            self.pool.allocator.incref(b)
            child.block_table.append(b)
        if parent.context_len % bs:
            nb = self.pool.allocator.alloc()
            self.pool.copy_block(parent.block_table[full], nb)
            child.block_table.append(nb)
        self.slots.copy(parent.slot, child.slot)
        child.context_len = parent.context_len
        return child

    def reset(self) -> None:
        self.pool.allocator.reset()
        self.slots.reset()

    def _max_table_width(self) -> int:
        """Most pages one sequence can hold: the block-table width of the
        captured decode steps."""
        return min(self.pool.num_blocks, LatentCachePool.blocks_for(
            self.cfg.max_seq_length, self.pool.block_size))

    def _graph_for(self, rows: int) -> _DecodeGraph:
        padded = 1
        while padded < min(rows, 8):
            padded *= 2
        if rows > 8:
            padded = (rows + 7) // 8 * 8
        g = self._decode_graphs.get(padded)
        if g is None:
            g = self._decode_graphs[padded] = _DecodeGraph(self, padded)
        return g

    # ------------------------------------------------------ step planning

    def _plan(self, work, want):
        """Host-side layout of one step: takes the pages the new tokens
        need and returns (token ids, int metadata lists, wanted flat rows)."""
        bs = self.pool.block_size
        tokens, positions, tok_seq, page_slot, cu = [], [], [], [], [0]
        slot_idx, want_rows = [], []
        for b, (q, toks) in enumerate(work):
            n = len(toks)
            if n < 1:
                raise ValueError("every row of a step needs at least one token")
            p0 = q.context_len
            need = LatentCachePool.blocks_for(p0 + n, bs)
            while len(q.block_table) < need:
                q.block_table.append(self.pool.allocator.alloc())
            base = cu[-1]
            if n <= 8:
                for p in range(p0, p0 + n):
                    positions.append(p)
                    page_slot.append(q.block_table[p // bs] * bs + p % bs)
            else:
                p = torch.arange(p0, p0 + n, dtype=torch.int64)
                table = torch.tensor(q.block_table, dtype=torch.int64)
                positions.extend(p.tolist())
                page_slot.extend((table[p // bs] * bs + p % bs).tolist())
            tok_seq.extend([b] * n)
            tokens.extend(toks)
            cu.append(base + n)
            slot_idx.append(q.slot)
            for w in ([n - 1] if want is None else want[b]):
                if not 0 <= w < n:
                    raise ValueError("wanted place outside the row's tokens")
                want_rows.append(base + w)
        lengths = [len(t) for _, t in work]
        tiles, max_tile = SM.query_tiles(lengths)
        wide, max_wide = SM.query_tiles(lengths, SM.WIDE_QUERY_TILE)
        chunks, chunk_cu = SM.scan_chunks(lengths)
        meta = dict(positions=positions, tok_seq=tok_seq, page_slot=page_slot,
                    cu=cu, slots=slot_idx,
                    block_tables=[q.block_table for q, _ in work],
                    tiles=tiles, max_tile=max_tile, wide_tiles=wide,
                    max_wide_tile=max_wide, scan_chunks=chunks,
                    scan_cu=chunk_cu)
        return tokens, meta, want_rows

    @staticmethod
    def _pack(tokens, meta, want_rows, max_nb=None):
        """All int inputs of a step as one flat list (one host-to-device
        copy) plus the layout to cut it up again."""
        if max_nb is None:
            max_nb = max(len(t) for t in meta["block_tables"])
        flat, lay = [], {}
        tables = [v for t in meta["block_tables"]
                  for v in (t + [0] * (max_nb - len(t)))]
        tiles = [v for t in meta["tiles"] for v in t]
        for name, vals in (("tokens", tokens), ("positions", meta["positions"]),
                           ("tok_seq", meta["tok_seq"]),
                           ("page_slot", meta["page_slot"]), ("cu", meta["cu"]),
                           ("slots", meta["slots"]), ("block_tables", tables),
                           ("tiles", tiles),
                           ("wide_tiles", [v for t in meta.get("wide_tiles", [])
                                           for v in t]),
                           ("want", want_rows),
                           ("scan_chunks", [v for c in meta.get("scan_chunks", [])
                                            for v in c]),
                           ("scan_cu", meta.get("scan_cu", []))):
            lay[name] = (len(flat), len(vals))
            flat.extend(vals)
        lay["max_nb"] = max_nb
        lay["max_wide_tile"] = meta.get("max_wide_tile", 1)
        return flat, lay

    @staticmethod
    def _views(buf, lay, max_tile):
        def cut(name):
            a, n = lay[name]
            return buf[a:a + n]
        meta = {k: cut(k) for k in ("positions", "tok_seq", "page_slot", "cu",
                                    "slots")}
        meta["block_tables"] = cut("block_tables").view(-1, lay["max_nb"])
        meta["tiles"] = cut("tiles").view(-1, 3)
        meta["wide_tiles"] = cut("wide_tiles").view(-1, 3)
        meta["max_wide_tile"] = lay["max_wide_tile"]
        meta["scan_chunks"] = cut("scan_chunks").view(-1, 3)
        meta["scan_cu"] = cut("scan_cu")
        meta["max_tile"] = max_tile
        return cut("tokens").long(), meta, cut("want").long()

    # --------------------------------------------------------------- step

    @torch.no_grad()
    def step(self, work: List[Tuple[Sequence, Seq[int]]],
             want: Optional[List[Seq[int]]] = None,
             capture: Optional[list] = None) -> torch.Tensor:
        """Run the next tokens of every listed sequence as one flat batch.

        work: (sequence, its next tokens) rows, each with >= 1 token.
        want: per row, the places among its tokens whose logits are
        returned (default: the last one). Returns fp32 [sum(want), vocab]
        in row order. ``capture`` (a list) receives the residual stream
        after every layer."""
        tokens, meta, want_rows = self._plan(work, want)
        dev = self.device
        if (capture is None and dev.type == "cuda" and not self.cfg.enforce_eager
                and meta["max_tile"] == 1 and want_rows == list(range(len(work)))
                and max(len(t) for t in meta["block_tables"])
                <= self._max_table_width()):
            # decode-only step: replay the captured step of this batch size
            # (the graph's output buffer is reused by the next replay)
            logits = self._graph_for(len(work)).run(tokens, meta).clone()
            for q, toks in work:
                q.context_len += len(toks)
            return logits
        packed, lay = self._pack(tokens, meta, want_rows)
        buf = torch.tensor(packed, dtype=torch.int32).to(dev)
        tok_t, meta_t, want_t = self._views(buf, lay, meta["max_tile"])
        logits = self._forward(tok_t, meta_t, want_t, capture)
        for q, toks in work:
            q.context_len += len(toks)
        return logits

    # ---- mixers: (unit key, spec, weights, mixer input, step metadata) ->
    # [T, width]. ``proj`` carries the unit's rows of a projection the caller
    # already made (the sides of a parallel pair share one GEMM); ``x32`` is
    # the fp32 form of the mixer input where a block has one.

    def _const(self, key, make):
        """Small per-unit device constants (frequency tables, slopes)."""
        c = self._consts.get(key)
        if c is None:
            c = self._consts[key] = make()
        return c

    def _mix_latent(self, i, m, L, hm, meta, proj=None, x32=None):
        S, dt, T = self.spec, self.dtype, hm.shape[0]
        own = m.kv_from is None
        if proj is None:
            proj = F.linear(hm, L.in_w)
        cache = self.pool.unit_rows(i, m)
        nq = m.q_rank if m.q_rank else m.q_size
        if m.q_rank:
            # queries through a normed latent
            _, cq = SM.offset_rmsnorm(proj[:, :nq], L.q_norm_w, S.norm_eps, dt, 0.0)
            q = F.linear(cq, L.uq)
        else:
            q = proj[:, :nq]
        dkv = proj[:, nq:nq + m.cache_width] if own else None
        gate = None
        if m.out_gate:
            g0 = nq + (m.cache_width if own else 0)
            gate = proj[:, g0:g0 + m.heads]
        freqs, mag = None, 1.0
        if m.rope_pairs or m.rope_scaling:
            f, mag = m.rope_table()
            freqs = self._const(("rope", i), lambda: torch.tensor(
                f, dtype=torch.float64).to(torch.float32).to(self.device))
        q_rot = SM.latent_prepare(
            q, dkv, m.heads, m.dim, m.rot_dim, m.kv_rank,
            L.latent_norm_w if own else None, S.norm_eps, meta["positions"],
            m.rope_base, m.rope_dims, meta["page_slot"], cache, freqs, mag,
            m.rope_pairs)
        q_nope = q.view(T, m.heads, m.dim + m.rot_dim)
        q_lat = torch.bmm(q_nope[..., :m.dim].transpose(0, 1), L.uk)
        o_lat = SM.latent_window_attention(
            q_lat, q_rot, cache, m.kv_rank, meta["block_tables"],
            self.pool.block_size, meta["cu"], meta["tok_seq"],
            meta["positions"], m.window, m.scale, dt,
            tiles=meta["tiles"], max_tile=meta["max_tile"],
            sink=L.sink if m.sink else None, gate=gate)
        v = torch.bmm(o_lat, L.uv.transpose(1, 2))
        return F.linear(v.transpose(0, 1).reshape(T, m.heads * m.vdim), L.out_w)

    def _mix_mingru(self, i, m, L, hm, meta, proj=None, x32=None):
        zxg = F.linear(hm, L.in_w) if proj is None else proj
        a = SM.mingru_scan(zxg, L.in_b, self.slots.recurrent[i], meta["cu"],
                           meta["slots"], self.dtype, meta["scan_chunks"],
                           meta["scan_cu"])
        return F.linear(a, L.out_w)

    def _mix_sink_attention(self, i, m, L, hm, meta, shared, proj=None):
        """``shared`` carries the first value-mixing layer's fresh values of
        this step's tokens to the later mixing layers."""
        if proj is None:
            proj = F.linear(hm, L.in_w)
        cache = self.pool.unit_rows(i, m)
        v_first = shared.get(("v", m.v_first)) if m.v_first is not None else None
        q = SM.rope_kv_write(proj, m.heads, m.kv_heads, m.dim, m.vdim,
                             meta["positions"], m.rope_base, m.rope_dims,
                             meta["page_slot"], cache, L.vmix, v_first)
        if m.v_mix and m.v_first is None:
            shared[("v", i)] = proj[:, m.q_size + m.k_size:]
        o = SM.sink_attention(q, cache, m.heads, m.kv_heads, m.dim, m.vdim,
                              meta["block_tables"], self.pool.block_size,
                              meta["cu"], meta["tok_seq"], meta["positions"],
                              m.scale, m.softcap, L.sink, L.talk, self.dtype,
                              tiles=meta["wide_tiles"],
                              max_tile=meta["max_wide_tile"])
        return F.linear(o, L.out_w)

    def _mix_sigmoid_attention(self, i, m, L, hm, meta, proj=None, x32=None):
        if proj is None:
            proj = F.linear(hm, L.in_w)
        cache = self.pool.unit_rows(i, m)
        q = SM.qk_norm_kv_write(proj, m.heads, m.kv_heads, m.dim, m.vdim,
                                L.q_norm_w, L.k_norm_w, self.spec.norm_eps,
                                meta["page_slot"], cache)
        slopes = self._const(("slopes", i), lambda: torch.tensor(
            m.slopes(), dtype=torch.float64).to(torch.float32).to(self.device))
        o = SM.sigmoid_attention(q, cache, m.heads, m.kv_heads, m.dim, m.vdim,
                                 meta["block_tables"], self.pool.block_size,
                                 meta["cu"], meta["tok_seq"], meta["positions"],
                                 m.scale, m.window, m.keep_first, slopes,
                                 L.pos_bias, self.dtype,
                                 tiles=meta["wide_tiles"],
                                 max_tile=meta["max_wide_tile"])
        return F.linear(o, L.out_w)

    def _mix_window_attention(self, i, m, L, hm, meta, proj=None, x32=None):
        """Windowed softmax attention. Biases come with the projection GEMM;
        q/k norm, rotation, the fold of the score-mixing matrix into the
        queries and the page write are one kernel; distance bias, window,
        softmax and output gate are the attention kernel's."""
        if proj is None:
            proj = F.linear(hm, L.in_w, L.in_b if m.qkv_bias else None)
        cache = self.pool.unit_rows(i, m)
        freqs, mag = None, 1.0
        if m.rope_dims:
            f, mag = m.rope_table()
            freqs = self._const(("rope", i), lambda: torch.tensor(
                f, dtype=torch.float64).to(torch.float32).to(self.device))
        q = SM.qk_prepare_kv_write(
            proj, m.heads, m.kv_heads, m.dim, m.vdim,
            L.q_norm_w if m.qk_norm else None, L.k_norm_w if m.qk_norm else None,
            self.spec.norm_eps, meta["positions"], freqs, mag,
            L.talk if m.score_mix else None, meta["page_slot"], cache)
        gate = None
        if m.out_gate:
            g0 = m.q_size + m.k_size + m.v_size
            gate = proj[:, g0:g0 + m.heads]
        o = SM.window_attention(
            q, cache, m.heads, m.kv_heads, m.dim, m.vdim, m.score_mix,
            meta["block_tables"], self.pool.block_size, meta["cu"],
            meta["tok_seq"], meta["positions"], m.scale, m.window,
            m.keep_first, L.dist_r1 if m.log_distance else None,
            L.dist_r2 if m.log_distance else None, gate, self.dtype,
            tiles=meta["wide_tiles"], max_tile=meta["max_wide_tile"])
        return F.linear(o, L.out_w)

    def _mix_delta(self, i, m, L, hm, meta, proj=None, x32=None):
        if proj is None:
            proj = F.linear(hm, L.in_w)
        C = m.conv_channels
        qkv = SM.tap_conv_silu(proj[:, :C], L.conv_w, self.slots.mixer_tails[i],
                               meta["cu"], meta["tok_seq"], meta["slots"],
                               self.dtype)
        gate = proj[:, C:C + (m.gate_rank or m.v_size)]
        if m.gate_rank:
            gate = F.linear(gate, L.gate_up)
        # fp32 strength / decay inputs: read from the fp32 mixer input where
        # the block has one. Per-head decays: a GEMM for prompt-sized steps,
        # steps of a few tokens project them inside the op (two launches
        # fewer); per-channel decays always take the GEMM.
        if x32 is not None:
            ab, own = F.linear(x32, L.ab_w), {}
        elif m.decay == "channel" or hm.shape[0] > 256:
            ab, own = F.linear(hm.float(), L.ab_w), {}
        else:
            ab, own = None, dict(h=hm, ab_w=L.ab_w)
        o = SM.gated_delta_rule(qkv, gate, ab, L.a_log, L.dt_bias,
                                L.onorm_w, self.spec.norm_eps,
                                self.slots.recurrent[i], meta["cu"],
                                meta["slots"], m.heads, m.kv_heads, m.dim,
                                m.vdim, self.dtype,
                                decay_up=(L.decay_up if m.decay == "channel"
                                          else None),
                                gate_sigmoid=(m.gate == "sigmoid"), **own)
        return F.linear(o, L.out_w)

    def _mix_unit(self, key, m, W, hm, meta, shared, proj=None, x32=None):
        if isinstance(m, LatentAttentionSpec):
            return self._mix_latent(key, m, W, hm, meta, proj, x32)
        if isinstance(m, SinkAttentionSpec):
            return self._mix_sink_attention(key, m, W, hm, meta, shared, proj)
        if isinstance(m, SigmoidAttentionSpec):
            return self._mix_sigmoid_attention(key, m, W, hm, meta, proj, x32)
        if isinstance(m, WindowAttentionSpec):
            return self._mix_window_attention(key, m, W, hm, meta, proj, x32)
        if isinstance(m, DeltaRuleSpec):
            return self._mix_delta(key, m, W, hm, meta, proj, x32)
        return self._mix_mingru(key, m, W, hm, meta, proj, x32)

    def _mixer(self, i, ls, L, hm, meta, shared, x32=None):
        """-> (output, second output or None, their scales)."""
        m = ls.mixer
        if isinstance(m, ParallelMixerSpec):
            proj = F.linear(hm, L.in_w)
            nl = m.left.in_size
            left = self._mix_unit((i, 0), m.left, L.left, hm, meta, shared,
                                  proj[:, :nl], x32)
            right = self._mix_unit((i, 1), m.right, L.right, hm, meta, shared,
                                   proj[:, nl:], x32)
            return left, right, (m.left_scale, m.right_scale)
        return self._mix_unit(i, m, L, hm, meta, shared, None, x32), None, (1.0, 1.0)

    # ---- feed-forwards: -> (main output, second addend or None)

    def _ff(self, f, L, hb):
        if isinstance(f, GluSpec):
            gu = F.linear(hb, L.gu_w)
            act = SM.silu_glu(gu) if f.act == "silu" else SM.capped_glu(gu, f.limit)
            return F.linear(act, L.down_w), None
        if isinstance(f, MlpSpec):
            return F.linear(SM.gelu_tanh(F.linear(hb, L.up_w)), L.down_w), None
        if f.routing == "sigmoid":
            idx, wts = SM.moe_route_sigmoid(hb, L.router_w, f.top)
            if f.scale_input:
                return SM.moe_experts_scaled_input(hb, idx, wts, L.exp_gu,
                                                   L.exp_down), None
            return SM.moe_experts(hb, idx, wts, L.exp_gu, L.exp_down), None
        if f.routing == "all":
            idx, wts = SM.moe_route_all(hb, L.router_w, L.correction, f.top,
                                        f.scale)
            y = SM.moe_experts_glu(hb, idx, wts, L.exp_gu, L.exp_down, f.limit)
            if f.shared is None:
                return y, None
            return y, F.linear(SM.capped_glu(F.linear(hb, L.shared_gu),
                                             f.shared.limit), L.shared_down)
        idx, wts = SM.moe_route(hb, L.router_w, L.router_b, f.top)
        return SM.moe_experts(hb, idx, wts, L.exp_gu, L.exp_down), None

    # ---- block arrangements

    def _forward(self, tokens, meta, want_rows, capture=None) -> torch.Tensor:
        S, M, dt = self.spec, self.model, self.dtype
        if S.block == "sandwich":
            x = self._layers_sandwich(tokens, meta, capture)
        elif S.block == "post_norm":
            x = self._layers_post_norm(tokens, meta, capture)
        elif S.block == "pre_norm":
            x = self._layers_pre_norm(tokens, meta, capture)
        else:
            x = self._layers_parallel_gated(tokens, meta, capture)
        if want_rows.numel() == 0:
            return torch.empty(0, S.vocab_size, dtype=torch.float32,
                               device=x.device)
        _, hb = SM.offset_rmsnorm(x[want_rows], M.final_norm_w, S.norm_eps, dt,
                                  S.norm_offset, S.norm_groups)
        logits = F.linear(hb, M.head).float()
        return logits * S.logit_scale if S.logit_scale != 1.0 else logits

    def _layers_parallel_gated(self, tokens, meta, capture):
        """One norm per layer feeds the mixer (through the block's short
        convolution) and the feed-forward; their outputs enter the residual
        through sigmoid gates."""
        S, M, dt = self.spec, self.model, self.dtype
        eps, mult = S.norm_eps, S.residual_mult
        shared = {}
        x, _ = SM.offset_rmsnorm(M.embed[tokens], M.embed_norm_w, eps, dt)
        h32, hb = SM.offset_rmsnorm(x, M.layers[0].norm_w, eps, dt)
        last = S.num_layers - 1
        for i, (ls, L) in enumerate(zip(S.layers, M.layers)):
            if S.conv_taps:
                hm = SM.causal_tap_conv(h32, L.conv_w, self.slots.tails[i],
                                        meta["cu"], meta["tok_seq"],
                                        meta["slots"], dt)
            else:
                hm = hb
            gates = F.linear(hb, L.gate_w)
            y = self._mixer(i, ls, L, hm, meta, shared)[0]
            f = None
            if ls.mlp is not None:
                f, f2 = self._ff(ls.mlp, L, hb)
                if f2 is not None:
                    f = f.float() + f2.float()
            if i < last:
                h32, hb = SM.gated_residual_norm(
                    x, y, f, gates, L.gate_b, mult, M.layers[i + 1].norm_w,
                    eps, dt)
            else:
                SM.gated_residual_add(x, y, f, gates, L.gate_b, mult)
            if capture is not None:
                capture.append(x.clone())
        return x

    def _layers_sandwich(self, tokens, meta, capture):
        """x += post(mixer(pre(x))), then x += post(ff(pre(x))): every
        sublayer has an offset RMS norm before and after it. The residual
        update, the sublayer's closing norm and the next opening norm are
        one kernel."""
        S, M, dt = self.spec, self.model, self.dtype
        eps = S.norm_eps
        shared = {}
        x = M.embed[tokens].float()
        _, hb = SM.offset_rmsnorm(x, M.layers[0].norm_w, eps, dt)
        last = S.num_layers - 1
        for i, (ls, L) in enumerate(zip(S.layers, M.layers)):
            y = self._mixer(i, ls, L, hb, meta, shared)[0]
            nxt = M.layers[i + 1].norm_w if i < last else None
            hb = SM.sandwich_residual_norm(
                x, y, None, L.post_w,
                L.ff_norm_w if ls.mlp is not None else nxt, eps, dt)
            if ls.mlp is not None:
                f, f2 = self._ff(ls.mlp, L, hb)
                hb = SM.sandwich_residual_norm(x, f, f2, L.ff_post_w, nxt, eps, dt)
            if capture is not None:
                capture.append(x.clone())
        return x

    def _layers_post_norm(self, tokens, meta, capture):
        """x += norm(mixer(x)), then x += norm(ff(x)): the sublayers read
        the residual itself (in the model dtype for the matrix products, in
        fp32 where a recurrence's inputs are formed) and only their output
        is normed. The closing norm, the residual sum and the copy of the
        new residual in the model dtype are one kernel; a parallel pair's
        two outputs are scaled and summed there as well."""
        S, M, dt = self.spec, self.model, self.dtype
        eps, off = S.norm_eps, S.norm_offset
        shared = {}
        x = M.embed[tokens].float()
        if S.embed_scale != 1.0:
            x = x * S.embed_scale
        hb = x.to(dt)
        for i, (ls, L) in enumerate(zip(S.layers, M.layers)):
            y, y2, (a, b) = self._mixer(i, ls, L, hb, meta, shared, x32=x)
            hb = SM.sandwich_residual_norm(x, y, y2, L.post_w, None, eps, dt,
                                           off, a, b, cast_next=True)
            if ls.mlp is not None:
                f, f2 = self._ff(ls.mlp, L, hb)
                hb = SM.sandwich_residual_norm(x, f, f2, L.ff_post_w, None, eps,
                                               dt, off, cast_next=True)
            if capture is not None:
                capture.append(x.clone())
        return x

    def _layers_pre_norm(self, tokens, meta, capture):
        """x += mixer(norm(x)), then x += ff(norm(x)): each sublayer reads a
        (grouped) RMS norm of the fp32 residual and its output is added as it
        is. The residual sum and the norm the next sublayer reads are one
        kernel."""
        S, M, dt = self.spec, self.model, self.dtype
        eps, off, ng = S.norm_eps, S.norm_offset, S.norm_groups
        shared = {}
        x = M.embed[tokens].float()
        if S.embed_scale != 1.0:
            x = x * S.embed_scale
        _, hb = SM.offset_rmsnorm(x, M.layers[0].norm_w, eps, dt, off, ng)
        last = S.num_layers - 1
        for i, (ls, L) in enumerate(zip(S.layers, M.layers)):
            y = self._mixer(i, ls, L, hb, meta, shared)[0]
            nxt = M.layers[i + 1].norm_w if i < last else None
            hb = SM.residual_add_norm(
                x, y, L.ff_norm_w if ls.mlp is not None else nxt, eps, dt, off, ng)
            if ls.mlp is not None:
                f, _ = self._ff(ls.mlp, L, hb)
                hb = SM.residual_add_norm(x, f, nxt, eps, dt, off, ng)
            if capture is not None:
                capture.append(x.clone())
        return x

    def score(self, ids: Seq[int]) -> torch.Tensor:
        """Teacher-forced logits of every position of one token sequence
        (fp32 [len, vocab]), run through a temporary sequence."""
        q = self.open_sequence()
        try:
            return self.step([(q, list(ids))], [list(range(len(ids)))])
        finally:
            self.close_sequence(q)

    # ----------------------------------------------------------- generate

    @torch.no_grad()
    def generate(self, prompts: List[List[int]], sp: SamplingParams,
                 eos_token_id: Optional[int] = None,
                 prefill_token_budget: Optional[int] = None,
                 stream_cb=None,
                 token_limits: Optional[List[List[int]]] = None,
                 cancel_check=None) -> List[List[List[int]]]:
        """Generate ``sp.n`` completions per prompt (same contract as the
        dense ``Engine.generate``: candidate order, EOS included when
        emitted, ``stream_cb(prompt, cand, new_ids)``, per-candidate
        ``token_limits``, ``cancel_check(prompt)`` polled every step)."""
        try:
            return self._generate_inner(prompts, sp, eos_token_id,
                                        prefill_token_budget, stream_cb,
                                        token_limits, cancel_check)
        except Exception:
            self.reset()   # a failed call strands its sequences; calls are serialized
            raise

    def _generate_inner(self, prompts, sp, eos, budget, stream_cb,
                        token_limits, cancel_check):
        if token_limits is not None:
            if len(token_limits) != len(prompts):
                raise ValueError("token_limits must have one list per prompt")
            for per in token_limits:
                if len(per) != sp.n or any(
                        not (1 <= int(v) <= sp.max_tokens) for v in per):
                    raise ValueError("each token_limits entry needs sp.n caps "
                                     f"in [1, {sp.max_tokens}]")
        if sp.n > self.slots.num_slots:
            raise ValueError(f"SamplingParams.n={sp.n} exceeds the engine's "
                             f"{self.slots.num_slots} state slots")
        if any(len(p) == 0 for p in prompts):
            raise ValueError("empty prompt")
        if sp.seed is not None:
            self.generator.manual_seed(int(sp.seed))
        budget = int(budget or self.cfg.step_token_budget)
        bs = self.pool.block_size
        max_total = self.cfg.max_seq_length
        blocks_for = LatentCachePool.blocks_for
        results = [[None] * sp.n for _ in prompts]
        waiting = list(range(len(prompts)))
        prefilling: List[Sequence] = []    # prompt not fully run yet
        running: List[Sequence] = []       # decoding candidates

        def worst_blocks(q):
            return blocks_for(min(len(q.prompt_ids) + sp.max_tokens, max_total), bs)

        def reserved_blocks():
            need = 0
            for q in running + prefilling:
                need += worst_blocks(q) - len(q.block_table)
            for q in prefilling:
                need += (sp.n - 1) * (worst_blocks(q) - len(q.prompt_ids) // bs)
            return need

        def admit():
            if cancel_check is not None:
                for pi in [p for p in waiting if cancel_check(p)]:
                    waiting.remove(pi)
                    results[pi] = [[] for _ in range(sp.n)]
            while waiting:
                pi = waiting[0]
                L = min(len(prompts[pi]), max_total - 1)
                worst = blocks_for(min(L + sp.max_tokens, max_total), bs)
                need = worst + (sp.n - 1) * (worst - L // bs)
                free_slots = self.slots.num_free - (sp.n - 1) * len(prefilling)
                if (need > self.pool.allocator.num_free - reserved_blocks()
                        or free_slots < sp.n):
                    break
                waiting.pop(0)
                prefilling.append(self.open_sequence(prompts[pi][:L], pi))

        def retire(q):
            results[q.parent_prompt][q.cand_index] = q.output_ids
            self.close_sequence(q)

        def accept(q, tok):
            """Append a sampled token; True if the candidate goes on."""
            q.output_ids.append(tok)
            if stream_cb is not None:
                stream_cb(q.parent_prompt, q.cand_index, [tok])
            done = ((eos is not None and tok == eos)
                    or len(q.output_ids) >= (q.max_tokens or sp.max_tokens)
                    or q.total_len >= max_total)
            if done:
                retire(q)
            return not done

        while waiting or prefilling or running:
            if cancel_check is not None:
                for q in [q for q in running if cancel_check(q.parent_prompt)]:
                    running.remove(q)
                    retire(q)
                for q in [q for q in prefilling if cancel_check(q.parent_prompt)]:
                    prefilling.remove(q)
                    results[q.parent_prompt] = [[] for _ in range(sp.n)]
                    self.close_sequence(q)
            admit()
            work, want, kinds = [], [], []
            left = budget
            for q in running:
                work.append((q, [q.output_ids[-1]]))
                want.append([0])
                kinds.append("decode")
                left -= 1
            for q in prefilling:
                if left <= 0 and work:
                    break
                rest = len(q.prompt_ids) - q.context_len
                n = min(rest, max(left, 1))
                work.append((q, q.prompt_ids[q.context_len:q.context_len + n]))
                want.append([n - 1] if n == rest else [])
                kinds.append("last" if n == rest else "part")
                left -= n
            if not work:
                if waiting:
                    raise MemoryError("cache or slot pool too small to admit "
                                      "any waiting prompt")
                break
            with trace_range(f"hybrid/step[{len(work)}]"):
                logits = self.step(work, want)
            # one sampler call: a finished prompt's row is drawn n times
            src, row = [], 0
            for k in kinds:
                if k != "part":
                    src += [row] * (sp.n if k == "last" else 1)
                    row += 1
            toks = OF.sample_tokens(
                logits[torch.tensor(src, dtype=torch.long, device=logits.device)]
                .contiguous(), sp.temperature, sp.top_p, sp.top_k,
                generator=self.generator).tolist() if src else []
            at = 0
            still = []
            for (q, _), kind in zip(work, kinds):
                if kind == "part":
                    continue
                if kind == "decode":
                    if accept(q, toks[at]):
                        still.append(q)
                    at += 1
                    continue
                prefilling.remove(q)
                cands = [q] + [self.fork_sequence(q) for _ in range(sp.n - 1)]
                for ci, c in enumerate(cands):
                    c.cand_index = ci
                    if token_limits is not None:
                        c.max_tokens = int(token_limits[q.parent_prompt][ci])
                    if accept(c, toks[at + ci]):
                        still.append(c)
                at += sp.n
            running = still
        return results
