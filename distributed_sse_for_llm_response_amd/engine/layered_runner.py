"""Forward passes of configuration-driven designs (models/muderax.py) on the layer-mechanism kernels (ops/layers.py).

A step is a set of packed rows -- the B decode slots first (one row each, state on the device as in ModelRunner), then
the rows of prompt portions -- that walk the layer list once:

    embed_rows              stream (fp32) = embedding; xb = its rounding (what the projections read)
    latent_attention layer  q and down-projection GEMMs -> latent_kv_write (norm + rotation + paged cache row) -> per-head
                            fold of the unrotated query through the key up-projection -> latent_attention over the
                            window (decode slots: one-row items; portions: tiled items) -> per-head value up-projection
                            -> output GEMM (fp32)
    rglru layer             gelu-branch and input GEMMs (fp32 out) -> conv_state (+ input bias; slot tail) -> block-
                            diagonal gate GEMM -> lru_scan (coefficients for all rows at once, then the walk over each
                            sequence's rows with the branch's bias + gelu; slot state) -> output GEMM (fp32)
    feed-forward            router GEMM (fp32 logits) -> moe_topk -> moe_grouped (rows sorted by expert, 16-row MFMA tiles; the shared expert is one
                            more slot of every row) -> per-slot outputs, summed inside the norm
    after each sublayer     scalar_norm: stream += out / rms(out) * g; xb = rounding
    head                    scalar_norm (final) on the rows that need logits -> GEMM (fp32 logits)

The residual stream, norms, scores, router and recurrence are fp32 in both element types; ``dtype=torch.float32`` runs
the projections in true fp32 as well (the exact mode).  The cache is paged with the engine's block tables and
allocator (LatentKVCache); recurrent layers keep their state in the sequence's decode slot (RecurrentStateCache), so
slots and pages are handed from one sequence to the next with no clearing pass.  The decode step of each batch bucket
is captured into a graph like ModelRunner's; prompt portions and mixed steps run eagerly.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .. import ops
from ..models.muderax import LRU_DECAY_SCALE
from ..parallel.comm import TPComm
from .kv_cache import PAGE, LatentKVCache, RecurrentStateCache
from .model_runner import RunnerBase, _capture, batch_buckets
from .weights import LayeredWeights

ATTN_ROWS_TILE = 4    # query rows per work item of the row-wise attention kernel (prompt portions)
FLASH_DECODE_WAVES = 512  # waves a decode attention launch aims for (two per CU)
FLASH_ROWS_TILE = 4   # query rows per work item of the MFMA attention form, x 4 heads = 16 columns: a page of keys is
                      # read once for four heads (16 rows x 1 head re-read it per head: 2-3x the time at 16 heads)


class LayeredRunner(RunnerBase):
    def __init__(self, w: LayeredWeights, num_blocks: int, max_batch: int = 64, max_model_len: int = 4096,
                 max_prefill_tokens: int = 8192, device="cuda", comm: TPComm | None = None, use_graphs=None):
        self.w, self.cfg = w, w.cfg
        self.device = torch.device(device)
        self.comm = comm or TPComm()
        if self.comm.size != 1:
            raise ValueError(f"{self.cfg.name}: tensor parallelism is not implemented for this family")
        self.dtype = w.dtype
        self.max_batch = max_batch
        self.max_model_len = max_model_len
        self.max_blocks = math.ceil(max_model_len / PAGE) + 1
        self.max_prefill_tokens = max_prefill_tokens
        self.use_graphs = (self.device.type == "cuda") if use_graphs is None else use_graphs
        cfg, dev = self.cfg, self.device
        self._init_slots(max_batch, self.max_blocks, cfg.vocab_size, dev, self.comm)
        att = {i: L.mixer for i, L in enumerate(cfg.layers) if L.kind == "latent_attention"}
        rec = {i: L.mixer for i, L in enumerate(cfg.layers) if L.kind == "rglru"}
        flash = {i: m.kv_rank for i, m in att.items() if ops.latent_flash_ok(self.dtype, m.kv_rank, m.rot_dim)}
        self.kv = LatentKVCache({i: m.kv_rank + m.rot_dim for i, m in att.items()}, num_blocks, dev, self.dtype,
                                transposed=flash)
        self.state = RecurrentStateCache({i: (m.width, m.conv) for i, m in rec.items()}, max_batch, dev)
        # one rotation table per distinct (rotation, rotated width)
        self._rope = {}
        for m in att.values():
            key = (m.rot, m.rot_dim)
            if key not in self._rope:
                self._rope[key] = m.rot.table(max_model_len + 1, m.rot_dim, dev)
        self._dec = self._buffers(max_batch)  # static decode activations (captured graphs read and write them)
        words = max((ops.latent_flash_part_floats(max_batch, m.heads, 16, 16, m.kv_rank) for i, m in att.items()
                     if i in flash), default=0)
        self._flash_part = torch.zeros(max(1, words), device=dev, dtype=torch.float32)

    # ------------------------------------------------------------------ buffers
    def _buffers(self, M: int) -> dict:
        cfg, dev = self.cfg, self.device
        f32 = dict(device=dev, dtype=torch.float32)
        el = dict(device=dev, dtype=self.dtype)
        W = cfg.width
        d = {"resid": torch.zeros(M, W, **f32), "xb": torch.zeros(M, W, **el), "y": torch.zeros(M, W, **f32)}
        att = [L.mixer for L in cfg.layers if L.kind == "latent_attention"]
        rec = [L.mixer for L in cfg.layers if L.kind == "rglru"]
        moe = [L.mlp for L in cfg.layers if L.mlp is not None]
        if att:
            d["q"] = torch.zeros(M * max(m.heads * (m.dim + m.rot_dim) for m in att), **el)
            d["ckr"] = torch.zeros(M * max(m.kv_rank + m.rot_dim for m in att), **f32)
            d["qabs"] = torch.zeros(M * max(m.heads * m.kv_rank for m in att), **f32)
            d["lat"] = torch.zeros(M * max(m.heads * m.kv_rank for m in att), **el)
            d["attn"] = torch.zeros(M * max(m.heads * m.vdim for m in att), **el)
        if rec:
            C = max(m.width for m in rec)
            d["ub"], d["hs"] = (torch.zeros(M * C, **el) for _ in range(2))
            d["yr"], d["ux"], d["u"] = (torch.zeros(M * C, **f32) for _ in range(3))
            d["gates"] = torch.zeros(M * 2 * C, **f32)
            # chunked walk of the recurrence over prompt portions: (A, B) per 32-row chunk
            d["scan"] = torch.zeros(2 * (M // 32 + max(M, self.max_batch) + 2) * C, **f32) if M >= 128 else None
        if moe:
            top = max(f.top for f in moe)
            d["tki"] = torch.zeros(M * top, device=dev, dtype=torch.int32)
            d["tkw"] = torch.zeros(M * top, **f32)
            # grouped experts: ids = (row, slot), slots = top (+ 1: the shared expert)
            slots = max(f.top + (1 if f.shared_ff else 0) for f in moe)
            tiles = -(-M * slots // 64) + max(f.experts for f in moe) + 2
            d["mo_z"] = torch.zeros(M * max(f.experts for f in moe), **f32)
            ldh = -(-max(max(f.ff, f.shared_ff) for f in moe) // 8) * 8
            d["mo_sorted"] = torch.zeros(tiles * 64, device=dev, dtype=torch.int32)
            d["mo_tile"] = torch.zeros(tiles, device=dev, dtype=torch.int32)
            d["mo_n"] = torch.zeros(1, device=dev, dtype=torch.int32)
            d["mo_h"] = torch.zeros(M * slots, ldh, **el)
            d["mo_o"] = torch.zeros(M * slots * W, **f32)
        return d

    # ------------------------------------------------------------------ layers
    @staticmethod
    def _lin(x, w, wt, out) -> None:
        """out = x · Wᵀ: the engine's tiled-layout GEMMs when the projection was tiled at load (model-sized, aligned
        shapes: weights.fits_tiled), else the general row-major GEMM."""
        if wt is not None:
            ops.gemm_out(x, wt, out)
        else:
            ops.gemm_rm(x, w, out)

    def _attention(self, li: int, m, Lw, M: int, d: dict, pos, slots, groups: list) -> None:
        H, dn, dr, rk, dv = m.heads, m.dim, m.rot_dim, m.kv_rank, m.vdim
        rope = self._rope[(m.rot, m.rot_dim)]
        cache = self.kv[li]
        q = d["q"][:M * H * (dn + dr)].view(M, H, dn + dr)
        ckr = d["ckr"][:M * (rk + dr)].view(M, rk + dr)
        qabs = d["qabs"][:M * H * rk].view(M, H, rk)
        lat = d["lat"][:M * H * rk].view(M, H, rk)
        attn = d["attn"][:M * H * dv].view(M, H, dv)
        self._lin(d["xb"], Lw.q, Lw.q_t, q.view(M, H * (dn + dr)))
        ops.gemm_rm(d["xb"], Lw.dkv, ckr)
        vt = self.kv.vt.get(li)
        ops.latent_kv_write(ckr, Lw.dkv_norm, pos, slots, rope, cache, self.cfg.eps, vt)
        ops.gemm_rm(q[:, :, :dn].permute(1, 0, 2), Lw.uk_t, qabs.permute(1, 0, 2))
        for g in groups:
            if vt is not None:  # MFMA form: a decode row's heads side by side, a portion's rows in tiles of 16
                dec = g["qt"] == 1
                if dec:  # few items: their keys are split over partitions so that the chip is filled
                    B = g["ws"].numel()
                    np_ = self._decode_parts(B, H, m.window)
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope,
                                         lat, m.window, m.scale, 1, vt, 16, self._flash_part if np_ > 1 else None, np_)
                else:
                    ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["fs"], g["ft"], rope,
                                         lat, m.window, m.scale, FLASH_ROWS_TILE, vt, 16 // FLASH_ROWS_TILE)
            else:
                ops.latent_attention(q, qabs, cache, g["bt"], g["qs"], g["ql"], g["ctx"], g["ws"], g["wt"], rope, lat,
                                     m.window, m.scale, g["qt"])
        ops.gemm_rm(lat.permute(1, 0, 2), Lw.uv, attn.permute(1, 0, 2))
        self._lin(attn.view(M, H * dv), Lw.o, Lw.o_t, d["y"])

    def _decode_parts(self, B: int, heads: int, window: int) -> int:
        """Key partitions of the decode attention: enough (item, head tile, partition) waves for the chip, at most one
        per page that a sequence can hold inside the window, at most 16."""
        pages = -(-min(window, self.max_model_len) // PAGE) + 1
        want = -(-FLASH_DECODE_WAVES // max(1, B * (-(-heads // 16))))
        return max(1, min(16, pages, want))

    def _recurrent(self, li: int, m, Lw, M: int, d: dict, groups: list) -> None:
        C, nb = m.width, m.blocks
        bw = C // nb
        ub, hs = (d[k][:M * C].view(M, C) for k in ("ub", "hs"))
        yr, ux, u = (d[k][:M * C].view(M, C) for k in ("yr", "ux", "u"))
        gates = d["gates"][:M * 2 * C].view(M, nb, 2 * bw)
        # both input projections leave fp32 without bias: the convolution adds its input's bias, the scan applies
        # the branch's bias and gelu
        self._lin(d["xb"], Lw.y, Lw.y_t, yr)
        self._lin(d["xb"], Lw.x, Lw.x_t, ux)
        for g in groups:
            ops.conv_state(ux, Lw.conv, Lw.conv_b, self.state.tail[li], g["qs"], g["ql"], g["ctx"], g["ss"], u, ub,
                           Lw.x_b)
        ops.gemm_rm(ub.view(M, nb, bw).permute(1, 0, 2), Lw.gates, gates.permute(1, 0, 2), bias=Lw.gates_b)
        for i, g in enumerate(groups):
            scr = d.get("scan")
            if scr is not None:
                slots = M // 32 + g["ql"].numel() + 1
                scr = scr[:2 * slots * C].view(2, slots, C)
            ops.lru_scan(u, gates, yr, Lw.lam, self.state.state[li], g["qs"], g["ql"], g["ctx"], g["ss"], hs,
                         LRU_DECAY_SCALE, Lw.y_b, i == 0, scr)
        self._lin(hs, Lw.o, Lw.o_t, d["y"])

    def _moe(self, f, Fw, M: int, d: dict):
        """Router + grouped experts; returns (per-slot outputs [M * S, W] fp32, S): the norm that follows sums them."""
        tki = d["tki"][:M * f.top].view(M, f.top)
        tkw = d["tkw"][:M * f.top].view(M, f.top)
        S = f.top + (1 if f.shared_ff else 0)
        o = d["mo_o"][:M * S * self.cfg.width].view(M * S, self.cfg.width)
        z = d["mo_z"][:M * f.experts].view(M, f.experts)
        ops.gemm_rm(d["xb"], Fw.router, z, bias=Fw.router_b)  # fp32 logits
        ops.moe_topk(z, tki, tkw)
        ops.moe_grouped(d["xb"], tki, tkw, Fw.gate, Fw.up, Fw.down, Fw.sgate, Fw.sup, Fw.sdown, d["mo_sorted"],
                        d["mo_tile"], d["mo_n"], d["mo_h"], o)
        return o, S

    def _layers(self, M: int, d: dict, ids, pos, slots, groups: list, trace: list | None = None) -> None:
        """Embedding + every layer over M packed rows.  `groups`: sequence groups of the step (decode slots, prompt
        portions), each with its own metadata (block tables bt, q_start qs, q_len ql, ctx_len ctx, state slots ss,
        attention work items ws / wt of qt rows).  trace (a list) receives a copy of the stream after every layer."""
        cfg, eps = self.cfg, self.cfg.eps
        ops.embed_rows(ids, self.w.embed, d["resid"], d["xb"])
        for li, (L, Lw) in enumerate(zip(cfg.layers, self.w.layers)):
            if L.kind == "latent_attention":
                self._attention(li, L.mixer, Lw.mix, M, d, pos, slots, groups)
            else:
                self._recurrent(li, L.mixer, Lw.mix, M, d, groups)
            ops.scalar_norm(d["y"], Lw.norm1, d["resid"], d["xb"], eps)
            if L.mlp is not None:
                o, S = self._moe(L.mlp, Lw.mlp, M, d)
                ops.scalar_norm(o, Lw.norm2, d["resid"], d["xb"], eps, S)
            if trace is not None:
                trace.append(d["resid"].clone())

    def _lm_head(self, rows, logits) -> None:
        """rows: fp32 stream rows (not normed yet) -> final one-number norm -> head GEMM."""
        xn = torch.empty(rows.shape, device=rows.device, dtype=self.dtype)
        ops.scalar_norm(None, self.w.final_norm, rows.contiguous(), xn, self.cfg.eps)
        self._lin(xn, self.w.head, self.w.head_t, logits)

    # ------------------------------------------------------------------ decode
    def _decode_group(self, B: int) -> dict:
        r = slice(0, B)
        return {"bt": self.block_tables[r], "qs": self.q_start[r], "ql": self.q_len[r], "ctx": self.ctx_len[r],
                "ss": self.q_start[r], "ws": self.work_seq[r], "wt": self.work_tile[r], "qt": 1}

    def decode_forward(self, B: int) -> None:
        """One decode step over slots [0, B) (graph-capturable: fixed shapes, no host sync).  Inactive slots
        (q_len 0) write no cache row and touch no state."""
        r = slice(0, B)
        ops.decode_prep(self.active[r], self.positions[r], self.block_tables[r], self.slots[r], self.ctx_len[r],
                        self.q_len[r], self.kv.num_blocks)
        d = {k: (v[:B] if k in ("resid", "xb", "y") else v) for k, v in self._dec.items()}
        self._layers(B, d, self.ids[r], self.positions[r], self.slots[r], [self._decode_group(B)])
        xn = self._dec["xb"][:B]
        ops.scalar_norm(None, self.w.final_norm, d["resid"], xn, self.cfg.eps)
        self._lin(xn, self.w.head, self.w.head_t, self.logits[r])
        self._sample_commit(B)
        ops.ring_advance(self.ring_counter)

    def capture(self, buckets=None) -> None:
        """Capture the decode step of each batch bucket into its own graph (shared memory pool)."""
        if not self.use_graphs:
            return
        buckets = buckets or batch_buckets(self.max_batch)
        s = torch.cuda.Stream(self.device)
        s.wait_stream(torch.cuda.current_stream(self.device))
        saved = self._snapshot_state()
        act = self.active.clone()
        self.active.zero_()  # every slot inactive: the warm-up and capture runs touch no cache row and no state
        with torch.cuda.stream(s):
            for B in buckets:
                self.decode_forward(B)
        torch.cuda.current_stream(self.device).wait_stream(s)
        torch.cuda.synchronize(self.device)
        for B in sorted(buckets, reverse=True):
            g = torch.cuda.CUDAGraph()
            with _capture(g, pool=self.graph_pool):
                self.decode_forward(B)
            if self.graph_pool is None:
                self.graph_pool = g.pool()
            self.graphs[B] = g
        torch.cuda.synchronize(self.device)
        self.active.copy_(act)
        self._restore_state(saved)

    def move_slots(self, src: list, dst: list) -> None:
        """Slot compaction: last token and position (RunnerBase) and the recurrent state of each moved slot."""
        super().move_slots(src, dst)
        idx = torch.tensor([src, dst], dtype=torch.long)
        if self.device.type == "cuda":
            idx = idx.pin_memory().to(self.device, non_blocking=True)
        self.state.move(idx[0], idx[1])

    def close(self) -> None:
        pass

    # ------------------------------------------------------------------ prompt portions
    def _pack(self, seqs: list, row0: int = 0):
        """Packed metadata of prompt portions whose rows start at `row0`: one pinned upload.  Returns (T, q_start
        list, device dict: ids / pos / slots per row, qs / ql / ctx / ss per sequence, ws / wt work items, bt)."""
        n = len(seqs)
        ids_l, pos_l, slots_l, qs, ql, ctx, ss, ws, wt, fs, ft = [], [], [], [], [], [], [], [], [], [], []
        bt = torch.zeros(n, self.max_blocks, dtype=torch.int32)
        row = 0
        for i, s in enumerate(seqs):
            m = len(s.tokens)
            p = s.start_pos + np.arange(m, dtype=np.int64)
            table = np.asarray(s.block_table, dtype=np.int64)
            ids_l.append(np.asarray(s.tokens, dtype=np.int64))
            pos_l.append(p)
            slots_l.append(table[p // PAGE] * PAGE + p % PAGE)
            qs.append(row0 + row)
            ql.append(m)
            ctx.append(s.start_pos + m)
            ss.append(s.slot)
            bt[i, : len(s.block_table)] = torch.from_numpy(table.astype(np.int32))
            nt = math.ceil(m / ATTN_ROWS_TILE)
            ws += [i] * nt
            wt += list(range(nt))
            nf = math.ceil(m / FLASH_ROWS_TILE)
            fs += [i] * nf
            ft += list(range(nf))
            row += m
        T = row
        meta = torch.from_numpy(np.concatenate(ids_l + pos_l + slots_l + [np.asarray(qs + ql + ctx + ss + ws + wt + fs + ft,
                                                                                     dtype=np.int64)]).astype(np.int32))
        if self.device.type == "cuda":
            meta = meta.pin_memory().to(self.device, non_blocking=True)
            bt = bt.pin_memory().to(self.device, non_blocking=True)
        d, o = {}, 0
        for name, k in (("ids", T), ("pos", T), ("slots", T), ("qs", n), ("ql", n), ("ctx", n), ("ss", n),
                        ("ws", len(ws)), ("wt", len(ws)), ("fs", len(fs)), ("ft", len(fs))):
            d[name], o = meta[o:o + k], o + k
        d["bt"] = bt
        d["qt"] = ATTN_ROWS_TILE
        return T, qs, ql, d

    def prefill(self, seqs: list, ring_row: int, trace: list | None = None) -> None:
        """One packed batch of prompt portions.  Sequences whose last portion this is sample their first token into
        ids[slot] and ring[ring_row, slot]; portions that ask for logits (PrefillSeq.want) leave them in kept_logits."""
        if not seqs:
            return
        T, qs, ql, g = self._pack(seqs)
        d = self._buffers(T)
        self._layers(T, d, g["ids"], g["pos"], g["slots"], [g], trace)
        self._prefill_sample(seqs, d["resid"], qs, ql, ring_row)
        self._keep_logits(seqs, d["resid"], qs)

    def mixed(self, B: int, seqs: list, ring_row: int) -> None:
        """ONE forward over the decode slots [0, B) and the prompt portions `seqs` (rows B .. B + T - 1): the weights
        stream once for both.  The decode rows sample and commit as the decode step does, finishing portions sample
        their first token as prefill() does."""
        T, qs, ql, g = self._pack(seqs, row0=B)
        M = B + T
        r = slice(0, B)
        ops.decode_prep(self.active[r], self.positions[r], self.block_tables[r], self.slots[r], self.ctx_len[r],
                        self.q_len[r], self.kv.num_blocks)
        ids = torch.cat([self.ids[r], g["ids"]])
        pos = torch.cat([self.positions[r], g["pos"]])
        slots = torch.cat([self.slots[r], g["slots"]])
        d = self._buffers(M)
        self._layers(M, d, ids, pos, slots, [self._decode_group(B), g])
        self._lm_head(d["resid"][r], self.logits[r])
        self._sample_commit(B)
        ops.ring_advance(self.ring_counter)
        self._prefill_sample(seqs, d["resid"], qs, ql, ring_row)
        self._keep_logits(seqs, d["resid"], qs)
