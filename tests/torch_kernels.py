"""A test double for the engine's kernel set, written with plain torch operations.

It exists so that the host side of the engine (batch layout, block tables, page reuse, scheduling, replay)
can be exercised where there is no GPU.  It is handed to `Engine(..., kernels=TorchKernels())` by tests only;
the product never constructs it and has no fallback to it.  Each method states the contract of the HIP
kernel of the same name; the GPU tests hold the HIP kernels to these same contracts.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from ampere_kv_engine_amd.parts.base import KernelSet


def _round(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return x.to(dtype)


class TorchKernels(KernelSet):
    name = "torch-double"

    def __init__(self, fold_rows: int = 0, fold_many_rows: int = 0, rows_left: bool = False):
        """`fold_rows`: steps of up to this many rows let a branch's last product add itself to the residual sum and
        the next product norm its rows from the sums of squares left there, as the HIP kernel set does in decode
        steps (0: never).  `fold_many_rows`: steps of more rows, up to this many, do the same the way the HIP
        kernel set's mid-size products do: the adding product leaves the new rows times the next norm's weight, and
        the reading product divides its results by the rows' root mean square."""
        self.fold_rows = fold_rows
        self.fold_many_rows = fold_many_rows
        # steps of up to `fold_rows` rows too: the adding product leaves the rows times the next norm's weight where it
        # is told that weight, and the reader scales its results (what the HIP kernel set's decode products do)
        self.rows_left = rows_left

    def check_attention_sizes(self, q_heads, kv_heads, head_dim, page_size):
        if q_heads % kv_heads:
            raise ValueError("q_heads must be a multiple of kv_heads")

    # ---- token-wise ------------------------------------------------------------------------------------
    def embed(self, ids, table, out, ctx=None):
        """An id of -1 stands for the token chosen last for the row's request (word 1 of its slot)."""
        ids = ids.long().clone()
        words = getattr(ctx, "slot_words", None) if ctx is not None else None
        if words is not None:
            last = words[ctx.seq_slots.long()[ctx.seq_of_token.long()], 1].long()
            ids = torch.where(ids == -1, last, ids)
        out.copy_(table[ids].float())

    def step_prologue(self, ctx):
        """state[offset] = value for the step's (offset, value) pairs; word 0 of every request's slot = its length."""
        count = int(ctx.patch_count[0])
        assert count <= ctx.patch_room
        pairs = ctx.patches[:2 * count].view(count, 2).long()
        ctx.slot_state[pairs[:, 0]] = pairs[:, 1].int()
        ctx.slot_words[ctx.seq_slots.long(), 0] = ctx.seq_lens

    def add_rmsnorm(self, stream, delta, weight, eps, out):
        if delta is not None:
            stream += delta.float()
        normed = stream * torch.rsqrt((stream * stream).mean(-1, keepdim=True) + eps)
        out.copy_(_round(_round(normed, out.dtype).float() * weight, out.dtype))

    def rmsnorm(self, x, weight, eps, out):
        xf = x.float()
        normed = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
        out.copy_(_round(_round(normed, out.dtype).float() * weight, out.dtype))

    def rmsnorm_heads(self, x, weight, eps, out):
        self.rmsnorm(x, weight, eps, out)

    def copy_heads(self, x, out):
        out.copy_(x)

    def gather_rows(self, stream, pending, rows, out):
        picked = stream[rows.long()]
        if pending is not None:
            picked = picked + pending[rows.long()].float()
        out.copy_(picked)

    def prepare_linear(self, matrix):
        return matrix

    def linear(self, x, weight, out, bias=None):
        y = x.float() @ weight.float().T
        out.copy_((y if bias is None else y + bias.float()).to(out.dtype))

    def prepare_gated_linear(self, gate, up):
        return (gate, up)

    # ---- the residual sum and the norm inside the products (decode steps) -------------------------------
    def folds_norm(self, rows, hidden, dtype):
        return 0 < rows <= max(self.fold_rows, self.fold_many_rows) and dtype == torch.bfloat16

    def adds_to_stream(self, rows, weight, dtype, gain=None):
        if not isinstance(weight, torch.Tensor) or dtype != torch.bfloat16:
            return False
        if 0 < rows <= self.fold_rows:
            return True
        return gain is not None and rows <= self.fold_many_rows

    def add_to_stream(self, x, weight, stream, arena, bias=None, gain=None):
        from ampere_kv_engine_amd.parts.base import StreamSums
        rows, outs = x.shape[0], weight.shape[0]
        if rows <= self.fold_rows:
            sums = arena.take(((outs + 15) // 16, 16), torch.float32)
            self.linear_adds(x, weight, stream, sums, bias=bias)
            if not self.rows_left or gain is None:
                return StreamSums(sums)
            left = arena.take((rows, outs), x.dtype)
            left.copy_((stream * gain).to(x.dtype))
            return StreamSums(sums, rows=left, gain=gain)
        # many rows: the new rows times the next norm's weight, and three groups of partial sums per row
        y = torch.empty(rows, outs, dtype=x.dtype)
        self.linear(x, weight, y, bias)
        stream += y.float()
        sums = arena.take((3, (rows + 15) // 16 * 16), torch.float32)
        sums.zero_()
        for group, columns in enumerate(torch.arange(outs).chunk(3)):
            sums[group, :rows] = (stream[:, columns] ** 2).sum(-1)
        left = arena.take((rows, outs), x.dtype)
        left.copy_((stream * gain).to(x.dtype))
        return StreamSums(sums, rows=left, gain=gain)

    def scales_rows_in_product(self, rows, weight, dtype, sums):
        return sums.rows is not None and 0 < rows <= max(self.fold_rows, self.fold_many_rows) and dtype == torch.bfloat16

    def linear_rowscaled(self, x, sums, eps, weight, out, bias=None):
        rows, k = x.shape
        scale = torch.rsqrt(sums.sum(0)[:rows, None] / k + eps)
        if isinstance(weight, tuple):
            g, u = x.float() @ weight[0].float().T * scale, x.float() @ weight[1].float().T * scale
            out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))
        else:
            y = x.float() @ weight.float().T * scale
            out.copy_((y if bias is None else y + bias.float()).to(out.dtype))

    def norms_rows_in_product(self, rows, weight, dtype):
        matrix = weight[0] if isinstance(weight, tuple) else weight
        return isinstance(matrix, torch.Tensor) and self.folds_norm(rows, matrix.shape[1], dtype)

    def linear_adds(self, x, weight, stream, sums, bias=None):
        y = torch.empty(x.shape[0], weight.shape[0], dtype=x.dtype)
        self.linear(x, weight, y, bias)
        stream += y.float()
        rows, outs = stream.shape
        padded = torch.zeros(rows, sums.shape[0] * 16)
        padded[:, :outs] = stream
        sums.zero_()
        sums[:, :rows] = (padded * padded).view(rows, -1, 16).sum(-1).T

    def linear_scaled(self, stream, sums, norm_weight, eps, weight, out, bias=None):
        rows, k = stream.shape
        scale = torch.rsqrt(sums.sum(0)[:rows, None] / k + eps)
        normed = _round(_round(stream * scale, out.dtype).float() * norm_weight, out.dtype)
        if isinstance(weight, tuple):
            self.gated_linear(normed, weight, out)
        else:
            self.linear(normed, weight, out, bias)

    def gated_scratch(self, weight, rows, dtype):
        return None

    def gated_linear(self, x, weight, out, scratch=None):
        g, u = x.float() @ weight[0].float().T, x.float() @ weight[1].float().T
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    def swiglu(self, gate_up, out):
        inter = out.shape[-1]
        g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    # ---- position ----------------------------------------------------------------------------------------
    def rope_table(self, inv_freq, table):
        positions = torch.arange(table.shape[0], dtype=torch.float32, device=table.device)
        angles = positions[:, None] * inv_freq[None, :].float()
        table[..., 0] = angles.cos()
        table[..., 1] = angles.sin()

    def _rotate(self, x, positions, table):
        half = x.shape[-1] // 2
        cs = table[positions.long()]                      # [N, d/2, 2]
        cos, sin = cs[:, None, :, 0], cs[:, None, :, 1]
        lo, hi = x[..., :half].float(), x[..., half:].float()
        return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin), dim=-1)

    def rope(self, x, positions, table):
        x.copy_(self._rotate(x, positions, table).to(x.dtype))

    # ---- cache ---------------------------------------------------------------------------------------------
    def kv_write(self, k, v, slot_map, k_pages, v_pages):
        pages, kv_heads, page_size, d = k_pages.shape
        slots = slot_map.long()
        k_pages[slots // page_size, :, slots % page_size] = k          # keys   [pages, kv_heads, page_size, d]
        v_pages[slots // page_size, :, :, slots % page_size] = v       # values [pages, kv_heads, d, page_size]

    def qk_norm_rope_write(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages,
                           q_out, q_heads, kv_heads, head_dim):
        n = qkv.shape[0]
        q_size, kv_size = q_heads * head_dim, kv_heads * head_dim
        q = qkv[:, :q_size].reshape(n, q_heads, head_dim).float()
        k = qkv[:, q_size:q_size + kv_size].reshape(n, kv_heads, head_dim).float()
        v = qkv[:, q_size + kv_size:].reshape(n, kv_heads, head_dim)
        dtype = qkv.dtype
        if q_weight is not None:
            q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps)
            q = _round(q, dtype).float() * q_weight
            k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps)
            k = _round(k, dtype).float() * k_weight
        if table is not None:
            q = self._rotate(_round(q, dtype), positions, table)
            k = self._rotate(_round(k, dtype), positions, table)
        q_out.copy_(q.reshape(n, q_size).to(dtype))
        if slot_map is not None:
            self.kv_write(k.to(dtype), v, slot_map, k_pages, v_pages)

    def encode_and_attend(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q, ctx,
                          meta, q_heads, kv_heads, head_dim, scale, window, out):
        self.qk_norm_rope_write(qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q,
                                q_heads, kv_heads, head_dim)
        self.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out)

    def attention(self, q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out):
        page_size = k_pages.shape[2]
        group = q_heads // kv_heads
        table = meta.block_table.cpu()
        if getattr(meta, "rows", None) is not None:          # the persistent table: a row per slot
            table = table[meta.rows.cpu().long()]
        for r in range(ctx.num_seqs):
            first, last = ctx.host_q_start[r], ctx.host_q_start[r + 1]
            length = ctx.host_seq_lens[r]
            history = length - (last - first)
            lowest = 0 if window is None else max(0, history - window + 1)
            key_pos = torch.arange(lowest, length)
            pages = table[r][key_pos // page_size].long()
            assert (pages >= 0).all(), "attention would read a page that was given back"
            keys = k_pages[pages, :, key_pos % page_size].float()        # [S, kv_heads, d]
            values = v_pages[pages, :, :, key_pos % page_size].float()
            qs = q[first:last].reshape(last - first, q_heads, head_dim).float()
            q_pos = history + torch.arange(last - first)
            visible = key_pos[None, :] <= q_pos[:, None]
            if window is not None:
                visible &= key_pos[None, :] > q_pos[:, None] - window
            merged = torch.empty_like(qs)
            for head in range(q_heads):          # a head at a time: long histories' scores of all heads need not fit
                scores = (qs[:, head] @ keys[:, head // group].T) * scale
                scores = scores.masked_fill(~visible, -math.inf)
                merged[:, head] = scores.softmax(-1) @ values[:, head // group]
            out[first:last] = merged.reshape(last - first, q_heads * head_dim).to(out.dtype)

    # ---- sampling -----------------------------------------------------------------------------------------
    def sample(self, logits, temperature, seeds, draws, out):
        """temperature 0: the largest logit, ties to the lowest id.  Otherwise the Gumbel-max draw
        argmax(logits / t - log(-log(u))), u from Philox-4x32-10 keyed by the seed with counter (id, draw).
        A row with a NaN, or with nothing above -infinity, gives -1."""
        for row in range(logits.shape[0]):
            if torch.isnan(logits[row]).any() or not (logits[row] > -math.inf).any():
                out[row] = -1
                continue
            t = float(temperature[row]) if temperature is not None else 0.0
            scores = logits[row].double()
            if t > 0:
                seed = int(seeds[row])
                bits = philox_first(np.arange(logits.shape[1]), int(draws[row]), seed & 0xFFFFFFFF, seed >> 32)
                u = ((bits >> np.uint64(8)).astype(np.float64) + 0.5) * 2.0 ** -24
                scores = scores / t - torch.from_numpy(np.log(-np.log(u)))
            best = scores.max()
            out[row] = int((scores == best).nonzero()[0])

    def argmax(self, logits, out):
        self.sample(logits, None, None, None, out)

    def sample_slots(self, logits, ctx, out):
        """`sample` with every row's temperature (word 2, float bits), seed (words 3 and 4) and draw count (word 5)
        read from its request's slot; the chosen token goes to word 1 and the draw count rises by one."""
        words = ctx.slot_words
        slots = ctx.seq_slots.long()[ctx.seq_of_token.long()[ctx.logit_rows.long()]]
        assert len(set(slots.tolist())) == len(slots), "two wanted rows of one request"
        state = words[slots].cpu()
        temperature = state[:, 2].contiguous().view(torch.float32)
        seeds = (state[:, 3].long() & 0xFFFFFFFF) | ((state[:, 4].long() & 0xFFFFFFFF) << 32)
        chosen = torch.empty(len(slots), dtype=torch.int32)
        self.sample(logits.cpu(), temperature, seeds, state[:, 5], chosen)
        out.copy_(chosen)
        words[slots, 1] = chosen.to(words.device)
        words[slots, 5] += 1


def philox_first(c0, c1, k0, k1):
    """First output word of Philox-4x32-10 for counters (c0, c1, 0, 0) and key (k0, k1); c0 may be an array."""
    c0 = np.asarray(c0, dtype=np.uint64)
    c1 = np.full_like(c0, np.uint64(c1))
    c2, c3 = np.zeros_like(c0), np.zeros_like(c0)
    k0, k1 = np.uint64(k0), np.uint64(k1)
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0, p1 = np.uint64(0xD2511F53) * c0, np.uint64(0xCD9E8D57) * c2
        c0, c1, c2, c3 = (((p1 >> np.uint64(32)) ^ c1 ^ k0) & mask, p1 & mask,
                          ((p0 >> np.uint64(32)) ^ c3 ^ k1) & mask, p0 & mask)
        k0, k1 = (k0 + np.uint64(0x9E3779B9)) & mask, (k1 + np.uint64(0xBB67AE85)) & mask
    return c0
