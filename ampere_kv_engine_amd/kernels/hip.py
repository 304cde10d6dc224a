"""The engine's kernel set: thin, checking wrappers over the HIP library (`csrc/api.h`) loaded with ctypes.

Every method checks on the host that shapes, dtypes, contiguity and devices are what its kernel and grid assume
before anything is launched, because a kernel reading outside its operands can take the whole GPU down.  There is
no other implementation behind these methods: if the library cannot be built or loaded, construction fails.
"""

from __future__ import annotations

import ctypes

import torch

from ..csrc.build import ensure_attention, ensure_built
from ..parts.base import KernelSet

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
MAX_HEAD_DIM = 256


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


class KernelError(RuntimeError):
    pass


class PackedWeight:
    """A bfloat16 matrix [outs, k] re-laid for the matrix cores: tiles of 16 rows x 32 k, 1 KB each, stored
    [row tile][k tile][lane][8] with lane = (k chunk of 8) * 16 + row; rows and k beyond the matrix are zero.
    `paired` (an even number of row tiles): [pair of row tiles][k tile][2][lane][8] - the two tiles of a pair lie side
    by side at every k-tile, for kernels in which one wave always owns both and so streams one run of memory."""

    def __init__(self, matrix: torch.Tensor, keep_row_major: bool = False, paired: bool = False):
        outs, k = matrix.shape
        self.outs, self.k, self.paired = outs, k, paired
        self.row_major = matrix if keep_row_major else None   # what a library product reads
        self.n_tiles, self.k_tiles = (outs + 15) // 16, (k + 31) // 32
        padded = matrix
        if outs % 16 or k % 32:
            padded = torch.zeros((self.n_tiles * 16, self.k_tiles * 32), dtype=matrix.dtype, device=matrix.device)
            padded[:outs, :k] = matrix
        self.data = (padded.view(self.n_tiles, 16, self.k_tiles, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
                     .view(self.n_tiles, self.k_tiles, 512))
        if paired:
            if self.n_tiles % 2:
                raise KernelError("a paired packing takes an even number of row tiles")
            self.data = (self.data.view(self.n_tiles // 2, 2, self.k_tiles, 512).permute(0, 2, 1, 3).contiguous()
                         .view(self.n_tiles, self.k_tiles, 512))     # (the shape no longer says where a tile lies)
        self.dtype, self.device, self.shape = matrix.dtype, matrix.device, (outs, k)

    def unpack(self) -> torch.Tensor:
        """The matrix back in row-major order (for checks)."""
        data = self.data
        if self.paired:
            data = data.view(self.n_tiles // 2, self.k_tiles, 2, 512).permute(0, 2, 1, 3).reshape(self.n_tiles, self.k_tiles, 512)
        full = data.view(self.n_tiles, self.k_tiles, 4, 16, 8).permute(0, 3, 1, 2, 4)
        return full.reshape(self.n_tiles * 16, self.k_tiles * 32)[:self.outs, :self.k].contiguous()


class GatedWeight:
    """Gate and up matrices [inter, k] of a gated feed-forward as ONE packed matrix whose row tiles alternate:
    tile 2t holds gate rows 16t .. 16t + 15, tile 2t + 1 the up rows of the same features; the packing is `paired`,
    so the wave that owns both reads them as one run."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, keep_row_major: bool = False):
        inter, k = gate.shape
        self.inter, self.k = inter, k
        # what a library product reads: gate rows, then up rows
        self.stacked = torch.cat((gate, up), dim=0).contiguous() if keep_row_major else None
        paired = torch.stack((gate.view(inter // 16, 16, k), up.view(inter // 16, 16, k)), dim=1).reshape(2 * inter, k)
        self.packed = PackedWeight(paired, paired=True)

    def unpack(self) -> tuple[torch.Tensor, torch.Tensor]:
        paired = self.packed.unpack().view(self.inter // 16, 2, 16, self.k)
        return paired[:, 0].reshape(self.inter, self.k), paired[:, 1].reshape(self.inter, self.k)


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


class HipKernels(KernelSet):
    name = "hip-gfx950"
    OWN_SKINNY_ROWS = 64            # the most rows the engine's own decode product takes

    def __init__(self, device: torch.device | str = "cuda:0", library_products_above: int | None = 16,
                 product_choices: dict | None = None):
        """`library_products_above`: bfloat16 products of more rows than this go to the BLAS library (torch.mm),
        which then needs the matrices row-major beside their packing; None keeps the packing alone and every
        product in this library's own kernels.  `product_choices`: which kernel takes a product of 17..512 rows,
        `{(kind, outs, k, row bucket): "own" | "mid" | "library"}` - a table that was measured once
        (`measure_products`) or loaded from a file; a fixed rule decides what the table does not name.  Nothing is
        ever timed or decided inside a step, so two runs with the same table send every product the same way and
        give the same bits."""
        self.library_products_above = library_products_above
        self.product_choices: dict = dict(product_choices or {})
        self._products: dict = {}              # (kind, outs, k) -> a prepared weight of that shape, for measure_products
        self._spacer = None                    # the buffer whose reads precede every timed run
        self._packed_rows = None               # where activations are repacked for the engine's own product
        self._mid_partial = None               # the mid-size product's partial sums, where it cuts k over blocks
        self._mid_counters = None              # and its arrival counters (zero between launches)
        self._outgrown = []                    # workspaces that were replaced by larger ones: recorded steps may name them
        self.device = torch.device(device)
        if self.device.type == "cuda" and self.device.index is None:
            self.device = torch.device("cuda", 0)
        if self.device.type != "cuda":
            raise KernelError(f"the HIP kernels run on a GPU; device {self.device} is not one")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine computes with HIP kernels only and has no CPU path")
        path = ensure_built()
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as error:
            raise KernelError(f"the kernel library {path} could not be loaded: {error}") from error
        self.library_path = path
        self._attention_entry = {}      # head size -> entry point of that head size's attention library
        self._exchange_tiles, self._exchange_pieces, self._exchange_arrivals = 0, None, None
        self.decode_wave_target = 2048  # decode attention cuts the keys until about this many waves are at work,
        self.decode_min_segment = 128   # but into segments no shorter than this many keys (measured: 64 and 256 are slower)
        self.decode_max_splits = 128    # and no more than this many (four waves of the merge share them)
        self.share_prompt_tiles = True  # prompt portions: blocks of four waves share keys and values through LDS
        self.one_wave_per_head = False  # True: every attention goes to the plain kernel, a wave per (token, head)
        self.fresh_decode_tokens = True  # single tokens: norm, rotation and cache write inside the attention kernel
        self.cut_keys_on_device = True  # single tokens: segments of one size for all requests, worked out from the lengths
        self._plan_buffers = []         # where such cuts are written: one buffer per plan of a step
        self.norm_in_products = True    # steps of a few rows: the products that follow a norm compute it themselves
        self.wide_prompt_tiles = None   # such blocks with 32 columns per wave instead of 16: None = by the step's size
        self.split_prompt_keys = None   # prompt portions on one wave per tile and key segment: None = by the step's size
        self.pair_launch = True         # a step of single tokens and short portions: their attention as one launch,
        self.portions_beside_single_tokens = True   # or, where that does not fit, the portions' on a second stream
        self._beside_stream = None
        self._sample_workspace = None   # where a row's blocks leave their parts' best logits (see `_sample_parts`)
        self.compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        for name in ("akv_embed", "akv_add_rmsnorm", "akv_rmsnorm_rows", "akv_copy_rows", "akv_gather_rows",
                     "akv_swiglu", "akv_rope_table", "akv_rope", "akv_kv_write", "akv_qk_norm_rope_write",
                     "akv_linear_tiled", "akv_linear_packed", "akv_linear_packed_swiglu", "akv_linear_packed_normed",
                     "akv_pack_rows", "akv_linear_packed_static", "akv_linear_mid", "akv_linear_mid_workspace",
                     "akv_linear_mid_adds", "akv_linear_mid_rowscaled", "akv_linear_mid_bands", "akv_linear_mid_most_groups",
                     "akv_linear_adds", "akv_linear_scaled", "akv_linear_adds_rows", "akv_linear_rowscaled",
                     "akv_linear_decode_plan", "akv_read_probe",
                     "akv_attention_rows", "akv_decode_plan", "akv_sample", "akv_sample_slots", "akv_sample_parts",
                     "akv_step_prologue"):
            getattr(self.lib, name).restype = ctypes.c_int
        self._check_slot_layout()

    def _check_slot_layout(self) -> None:
        """The words of a request's slot are laid out once for the kernels (csrc/common.h) and once for the host
        (cache/slots.py): a library built from another layout would read a seed as a temperature, so it is refused."""
        from ..cache import slots
        layout = (ctypes.c_int * 8)()
        self.lib.akv_slot_layout(layout)
        host = (slots.SLOT_WORDS, slots.WORD_LENGTH, slots.WORD_LAST_TOKEN, slots.WORD_TEMPERATURE, slots.WORD_SEED_LOW,
                slots.WORD_SEED_HIGH, slots.WORD_DRAWS, slots.WORD_TAKEN)
        if tuple(layout) != host:
            raise KernelError(f"the kernel library lays a request's slot out as {tuple(layout)} (words, then the indices of "
                              f"length, last token, temperature, seed low, seed high, draws, taken); the host as {host}")

    # ---- helpers -----------------------------------------------------------------------------------------
    def _stream(self):
        """The current stream's handle (the raw getter spares the construction of a Stream object per launch)."""
        if _raw_stream is not None:
            return ctypes.c_void_p(_raw_stream(self.device.index))
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def _check(self, status: int, what: str) -> None:
        if status == 0:
            return
        if status == -1:
            raise KernelError(f"{what}: dtype not supported by the kernel")
        if status == -2:
            raise KernelError(f"{what}: sizes not supported by the kernel")
        raise KernelError(f"{what}: launch failed with HIP error {status}")

    def _dense(self, t: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape: tuple | None = None):
        # (called a thousand times in a step that is not replayed from a recording: the comparisons are the cheap ones)
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.get_device() != self.device.index:
            raise KernelError(f"{name} must be a tensor on {self.device}, got {getattr(t, 'device', type(t))}")
        if not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
        if shape is not None and t.shape != (shape if type(shape) is tuple else tuple(shape)):
            raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
        return t

    def check_attention_sizes(self, q_heads: int, kv_heads: int, head_dim: int, page_size: int) -> None:
        if head_dim % 16 or not 16 <= head_dim <= MAX_HEAD_DIM:
            raise KernelError(f"head_dim {head_dim} is not supported: the attention kernels take multiples of 16 "
                              f"from 16 to {MAX_HEAD_DIM}")
        if q_heads % kv_heads:
            raise KernelError(f"q_heads {q_heads} is not a multiple of kv_heads {kv_heads}")
        if page_size <= 0:
            raise KernelError(f"page_size {page_size} must be positive")

    # ---- token-wise --------------------------------------------------------------------------------------
    def embed(self, ids, table, out, ctx=None):
        """out[n] = table[ids[n]].  With the step's context, an id of -1 stands for the token chosen last for the row's
        request, which the sampler left in the request's slot."""
        tokens = ids.shape[0]
        self._dense(ids, "ids", torch.int32, (tokens,))
        self._dense(table, "table")
        vocab, hidden = table.shape
        self._dense(out, "out", torch.float32, (tokens, hidden))
        words = getattr(ctx, "slot_words", None) if ctx is not None else None
        seq_of_token = seq_slots = None
        if words is not None:
            seq_of_token, seq_slots = ctx.seq_of_token, ctx.seq_slots
            self._dense(words, "slot_words", torch.int32)
            self._dense(seq_of_token, "seq_of_token", torch.int32, (tokens,))
            self._dense(seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
            if max(ctx.host_seq_slots) >= words.shape[0]:
                raise KernelError("a request's slot lies outside the slot words")
        self._check(self.lib.akv_embed(_ptr(ids), _ptr(table), _code(table), _ptr(out), tokens, hidden, vocab,
                                       _ptr(seq_of_token), _ptr(seq_slots), _ptr(words), self._stream()), "embed")

    def step_prologue(self, ctx) -> None:
        """Applies what the step changes in the device's persistent integer state before anything reads it: the
        block-table entries of pages its requests were handed or gave back, and the requests' new lengths."""
        state = ctx.slot_state
        self._dense(state, "slot_state", torch.int32)
        self._dense(ctx.patches, "patches", torch.int32, (2 * ctx.patch_room,))
        self._dense(ctx.patch_count, "patch_count", torch.int32, (1,))
        self._dense(ctx.seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
        self._dense(ctx.seq_lens, "seq_lens", torch.int32, (ctx.num_seqs,))
        self._check(self.lib.akv_step_prologue(_ptr(state), ctypes.c_long(state.numel()), _ptr(ctx.patches),
                                               _ptr(ctx.patch_count), ctx.patch_room, _ptr(ctx.seq_slots),
                                               _ptr(ctx.seq_lens), ctx.num_seqs, self._stream()), "step_prologue")

    def add_rmsnorm(self, stream, delta, weight, eps, out):
        tokens, hidden = stream.shape
        self._dense(stream, "stream", torch.float32)
        self._dense(weight, "weight", torch.float32, (hidden,))
        self._dense(out, "out", None, (tokens, hidden))
        if delta is not None:
            self._dense(delta, "delta", out.dtype, (tokens, hidden))
        self._check(self.lib.akv_add_rmsnorm(_ptr(stream), _ptr(delta), _ptr(weight), ctypes.c_float(eps), _ptr(out),
                                             _code(out), tokens, hidden, self._stream()), "add_rmsnorm")

    def _rows_view(self, x, name):
        """x [tokens, heads, width] whose last two axes are dense; returns (tokens, heads, width, token_stride)."""
        if x.dim() != 3 or x.stride(2) != 1 or x.stride(1) != x.shape[2] or x.device != self.device:
            raise KernelError(f"{name} must be [tokens, heads, width] on {self.device} with dense heads, got shape "
                              f"{tuple(x.shape)} strides {x.stride()}")
        return x.shape[0], x.shape[1], x.shape[2], x.stride(0)

    def rmsnorm(self, x, weight, eps, out):
        rows, width = x.shape
        self._dense(x, "x")
        self._dense(weight, "weight", torch.float32, (width,))
        self._dense(out, "out", x.dtype, (rows, width))
        self._check(self.lib.akv_rmsnorm_rows(_ptr(x), ctypes.c_long(width), _ptr(weight), ctypes.c_float(eps),
                                              _ptr(out), _code(x), ctypes.c_long(rows), 1, width, self._stream()),
                    "rmsnorm")

    def rmsnorm_heads(self, x, weight, eps, out):
        tokens, heads, width, stride = self._rows_view(x, "x")
        self._dense(weight, "weight", torch.float32, (width,))
        self._dense(out, "out", x.dtype, (tokens, heads, width))
        self._check(self.lib.akv_rmsnorm_rows(_ptr(x), ctypes.c_long(stride), _ptr(weight), ctypes.c_float(eps),
                                              _ptr(out), _code(x), ctypes.c_long(tokens), heads, width,
                                              self._stream()), "rmsnorm_heads")

    def copy_heads(self, x, out):
        tokens, heads, width, stride = self._rows_view(x, "x")
        self._dense(out, "out", x.dtype, (tokens, heads, width))
        self._check(self.lib.akv_copy_rows(_ptr(x), ctypes.c_long(stride), _ptr(out), _code(x), ctypes.c_long(tokens),
                                           heads, width, self._stream()), "copy_heads")

    def gather_rows(self, stream, pending, rows, out):
        tokens, hidden = stream.shape
        wanted = rows.shape[0]
        self._dense(stream, "stream", torch.float32)
        self._dense(rows, "rows", torch.int32, (wanted,))
        self._dense(out, "out", torch.float32, (wanted, hidden))
        code = 0
        if pending is not None:
            self._dense(pending, "pending", None, (tokens, hidden))
            code = _code(pending)
        self._check(self.lib.akv_gather_rows(_ptr(stream), _ptr(pending), code, _ptr(rows), _ptr(out), wanted, hidden,
                                             tokens, self._stream()), "gather_rows")

    def read_probe(self, data: torch.Tensor, out: torch.Tensor | None = None, blocks: int | None = None) -> torch.Tensor:
        """Reads `data` once the way the decode products read their weights (a contiguous span per wave, loads marked
        as read-once) and returns the xor of its 32-bit words per block, int32 [blocks]: timed over memory that no cache
        holds, it says what a kernel that only reads can draw - the ceiling the products are measured against."""
        self._dense(data, "data", None)
        size = data.numel() * data.element_size()
        if size % 16:
            raise KernelError("the read probe takes a multiple of 16 bytes")
        blocks = blocks or 4 * self.compute_units
        if out is None:
            out = torch.empty(blocks, dtype=torch.int32, device=self.device)
        self._dense(out, "out", torch.int32, (blocks,))
        self._check(self.lib.akv_read_probe(_ptr(data), ctypes.c_long(size), _ptr(out), blocks, self._stream()), "read_probe")
        return out

    def prepare_linear(self, matrix: torch.Tensor):
        """bfloat16 matrices whose k is a multiple of 8 are packed for the MFMA kernels; others stay row-major and
        go through the plain tiled kernel."""
        if matrix.dtype == torch.bfloat16 and matrix.shape[1] % 8 != 0:
            self._warn_once(("k", matrix.shape[1]), f"a bfloat16 matrix of {matrix.shape[0]} x {matrix.shape[1]}: its inner width is no "
                            "multiple of 8, so its products run in the plain float32 kernel instead of the matrix cores "
                            "(correct, and many times slower)")
        if matrix.dtype == torch.bfloat16 and matrix.shape[1] % 8 == 0:
            weight = PackedWeight(matrix, keep_row_major=self.library_products_above is not None)
            self._products.setdefault(("linear", weight.outs, weight.k), weight)
            self._reserve_exchange(weight.n_tiles)
            return weight
        return matrix

    PACK_ROWS_ABOVE = 16            # the engine's own product of more rows than this reads repacked activations
    PACKED_ROWS_ELEMENTS = 64 * 65536

    def _operand_rows(self, x, rows: int, k: int):
        """What the engine's own product of up to 64 rows reads as x, and whether that is the repacked form.  With
        several tiles of 16 rows the 16-byte gathers of a row-major x keep the vector memory pipe busier than the
        weights do; one small kernel lays x out [tile of 16 rows][k / 8][16 rows][8] first (into one buffer that all
        products on the stream share in turn), and an operand of the product is then 1 KB of consecutive bytes."""
        if not self.PACK_ROWS_ABOVE < rows <= self.OWN_SKINNY_ROWS or (rows + 15) // 16 * 16 * k > self.PACKED_ROWS_ELEMENTS:
            return x, 0
        if self._packed_rows is None:
            self._packed_rows = torch.empty(self.PACKED_ROWS_ELEMENTS, dtype=torch.bfloat16, device=self.device)
        self._check(self.lib.akv_pack_rows(_ptr(x), _ptr(self._packed_rows), rows, k, self._stream()), "pack_rows")
        return self._packed_rows, 1

    MID_ROWS = 512                  # the most rows the mid-size product takes

    @staticmethod
    def _row_bucket(rows: int):
        """Products of 17..512 rows are told apart by what the kernels make of the rows: tiles of 16 up to 64 rows
        (2, 3, 4), then blocks of 128 rows (8: up to 128; 16: up to 256; 32: up to 512)."""
        if rows <= 64:
            return (rows + 15) // 16
        return 8 if rows <= 128 else 16 if rows <= 256 else 32 if rows <= 512 else None

    def _route(self, kind: str, outs: int, k: int, rows: int, has_row_major: bool, out_dtype) -> str:
        """Which kernel takes a bfloat16 product of more than 16 rows: "own" (the skinny kernel up to 64 rows, the
        wide one above), "mid" (17..512 rows: the block's waves share the activations through LDS) or "library".
        The table of choices decides where it names the product; otherwise a fixed rule, from measurements at
        Qwen3-8B, -14B and -32B shapes (cold weights, 32 to 512 rows; `bench_products --rows ...` repeats them):
        plain products go to the mid-size kernel up to 256 rows (q/k/v, o, down at 128 rows: 26.8 / 21.6 / 36.8 us
        against the library's 28.5 / 27.4 / 69.7 at Qwen3-8B shapes, 36.9 / 31.8 / 70.1 against 44.6 / 47.2 / 185.7
        at Qwen3-32B's; the library's times jump with the row count), and up to 512 where k is at least twice the
        outputs (the down product: 69 against 84 us at 512 rows; the others are within a few percent either way
        there); the gated product up to 64 rows, and up to 128 where the two matrices hold no more than 64 M elements
        (Qwen3-8B: 47 against 57 us with the library's activation pass; Qwen3-14B: 100 / 101; Qwen3-32B: 126 / 112).
        Beyond, the library.  Without the library: the mid-size kernel up to 512 rows (it is faster than the skinny
        one from 17 rows on), the wide one beyond."""
        library = (has_row_major and self.library_products_above is not None and rows > self.library_products_above
                   and out_dtype == torch.bfloat16)
        bucket = self._row_bucket(rows)
        if bucket is None:
            return "library" if library else "own"
        choice = self.product_choices.get((kind, outs, k, bucket))
        if choice == "library" and not library:
            choice = None
        if choice is not None:
            return choice
        if not library:
            return "mid"
        if kind == "gated":
            return "mid" if rows <= 64 or (rows <= 128 and outs * k <= 64 << 20) else "library"
        if rows <= 256 or k >= 2 * outs:
            return "mid"
        return "library"

    def _mid(self, x, packed: PackedWeight, out, rows: int, outs: int, gated: bool, bias=None, adds=None, scaled=None) -> None:
        """The mid-size product (`csrc/gemm_mid.hip`).  Where it cuts k over blocks it needs room for partial sums
        and a few counters; both belong to this kernel set and serve one launch at a time (one stream).
        `adds` = (stream, gain, sums): the product adds itself to the residual sum (`add_to_stream`); `scaled` =
        (sums, eps): its results are divided by the rows' root mean square (`linear_rowscaled`)."""
        partial_floats, counters = ctypes.c_long(0), ctypes.c_long(0)
        self.lib.akv_linear_mid_workspace(rows, packed.n_tiles, packed.k_tiles, 1 if gated else 0, 0, 0, 0, 0,
                                          ctypes.byref(partial_floats), ctypes.byref(counters))
        if partial_floats.value:
            if self._mid_partial is None or self._mid_partial.numel() < partial_floats.value:
                if torch.cuda.is_current_stream_capturing():
                    raise KernelError("a recorded step needs more room for partial sums than the steps before it")
                self._outgrown.append(self._mid_partial)      # (a recorded step may still point at it)
                self._mid_partial = torch.empty(max(partial_floats.value, 8 << 20), dtype=torch.float32, device=self.device)
            if self._mid_counters is None or self._mid_counters.numel() < counters.value:
                if torch.cuda.is_current_stream_capturing():
                    raise KernelError("a recorded step needs more counters than the steps before it")
                self._outgrown.append(self._mid_counters)
                self._mid_counters = torch.zeros(max(counters.value, 1 << 16), dtype=torch.int32, device=self.device)
        held = lambda buffer: ctypes.c_long(buffer.numel() if buffer is not None else 0)
        if adds is not None:
            stream, gain, sums = adds
            self._check(self.lib.akv_linear_mid_adds(_ptr(x), _ptr(packed.data), _ptr(out), _ptr(self._mid_partial),
                                                     held(self._mid_partial), _ptr(self._mid_counters), held(self._mid_counters),
                                                     rows, outs, packed.k, packed.n_tiles, packed.k_tiles, _ptr(bias),
                                                     _ptr(stream), _ptr(gain), _ptr(sums), sums.shape[1], self._stream()),
                        "mid-size product that adds to the residual sum")
            return
        if scaled is not None:
            sums, eps = scaled
            self._check(self.lib.akv_linear_mid_rowscaled(_ptr(x), _ptr(packed.data), _ptr(out), _code(out), _ptr(self._mid_partial),
                                                          held(self._mid_partial), _ptr(self._mid_counters), held(self._mid_counters),
                                                          rows, outs, packed.k, packed.n_tiles, packed.k_tiles, 1 if gated else 0,
                                                          _ptr(bias), _ptr(sums), sums.shape[0], sums.shape[1],
                                                          ctypes.c_float(eps), self._stream()),
                        "mid-size product of rows to be scaled")
            return
        self._check(self.lib.akv_linear_mid(_ptr(x), _ptr(packed.data), _ptr(out), _code(out), _ptr(self._mid_partial),
                                            held(self._mid_partial), _ptr(self._mid_counters), held(self._mid_counters),
                                            rows, outs, packed.k, packed.n_tiles,
                                            packed.k_tiles, 1 if gated else 0, 0, 0, 0, 0, _ptr(bias), self._stream()),
                    "mid-size product")

    MEASURED_ROWS = (32, 48, 64, 128, 256, 512)

    def measure_products(self, rows_measured=MEASURED_ROWS, log=None) -> dict:
        """For every matrix shape prepared so far and a row count of every bucket from 17 to 512 rows: the kernels
        that can take the product ("own" up to 64 rows, "mid", "library" where there is one), each timed twice on the
        device; the fastest enters `product_choices`.  Before every timed run reads of 256 MB empty the caches, as the
        other layers' weights do in a real step, and keep the device busy while the host queues the run, so that
        the host's launch time is not part of what is measured.  Meant to be called once after loading
        (`EngineConfig.product_choices = "measure"`); returns the table, which `save_product_choices` writes for
        later runs.  Every decision is reported through `log` (default: the logger "ampere_kv_engine_amd.kernels")."""
        import logging
        report = log or logging.getLogger("ampere_kv_engine_amd.kernels").info
        if self._spacer is None:
            self._spacer = torch.zeros(64 << 20, dtype=torch.float32, device=self.device)
        for (kind, outs, k), weight in sorted(self._products.items(), key=lambda item: item[0]):
            for rows in rows_measured:
                bucket = self._row_bucket(rows)
                if rows <= 16 or bucket is None:
                    continue
                x = torch.randn(rows, k, device=self.device).to(torch.bfloat16)
                out = torch.empty(rows, outs, dtype=torch.bfloat16, device=self.device)
                row_major = weight.stacked if kind == "gated" else weight.row_major
                candidates = (["own"] if rows <= self.OWN_SKINNY_ROWS else []) + ["mid"]
                if row_major is not None and self.library_products_above is not None and rows > self.library_products_above:
                    candidates.append("library")
                scratch = torch.empty(rows, 2 * outs, dtype=torch.bfloat16, device=self.device) if kind == "gated" else None
                run = (lambda: self.gated_linear(x, weight, out, scratch)) if kind == "gated" else (lambda: self.linear(x, weight, out))
                best = {}
                for choice in candidates:
                    self.product_choices[kind, outs, k, bucket] = choice
                    run()                                            # (the first call may load code)
                    samples = []
                    for _ in range(2):
                        for _ in range(4):      # ~0.25 ms of device work: more than the host needs to queue what follows
                            self._spacer.sum()  # (reads: nothing is left to be written back while the run is timed)
                        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        start.record()
                        run()
                        end.record()
                        samples.append((start, end))
                    torch.cuda.synchronize(self.device)
                    best[choice] = min(a.elapsed_time(b) for a, b in samples)
                choice = min(best, key=best.get)
                self.product_choices[kind, outs, k, bucket] = choice
                report(f"product {kind} {outs}x{k}, {rows} rows: "
                       + ", ".join(f"{name} {time * 1000:.1f} us" for name, time in best.items()) + f" -> {choice}")
        return self.product_choices

    def save_product_choices(self, path: str) -> None:
        import json
        with open(path, "w") as handle:
            json.dump({f"{kind}:{outs}x{k}:{tiles}": choice
                       for (kind, outs, k, tiles), choice in sorted(self.product_choices.items())}, handle, indent=1)

    @staticmethod
    def load_product_choices(path: str) -> dict:
        """The table `save_product_choices` wrote: {"linear:6144x4096:2": "own", ...} -> {(kind, outs, k, bucket): choice}."""
        import json
        with open(path) as handle:
            raw = json.load(handle)
        table = {}
        for name, choice in raw.items():
            kind, shape, tiles = name.split(":")
            outs, k = shape.split("x")
            if choice not in ("own", "mid", "library"):
                raise ValueError(f"{path}: the choice for {name} is {choice!r}, not 'own', 'mid' or 'library'")
            table[kind, int(outs), int(k), int(tiles)] = choice
        return table

    def _bias(self, bias, outs: int):
        if bias is not None:
            self._dense(bias, "bias", torch.float32, (outs,))
        return bias

    def linear(self, x, weight, out, bias=None):
        """out = x W^T (+ bias): `bias` [outs] float32 is added to the float32 sums before they are rounded to
        `out`'s type - one rounding, as torch.nn.functional.linear makes."""
        if isinstance(weight, PackedWeight):
            rows, k = x.shape
            self._dense(x, "x", torch.bfloat16, (rows, weight.k))
            self._dense(out, "out", None, (rows, weight.outs))
            self._dense(weight.data, "packed weight", torch.bfloat16)
            self._bias(bias, weight.outs)
            route = "own" if rows <= 16 else self._route("linear", weight.outs, weight.k, rows,
                                                         weight.row_major is not None, out.dtype)
            if route == "library":
                if bias is None:
                    torch.mm(x, weight.row_major.t(), out=out)
                else:       # (the library adds the bias to its float32 sums too; it wants the bias in the result's type)
                    torch.addmm(self._library_bias(bias), x, weight.row_major.t(), out=out)
            elif route == "mid":
                self._mid(x, weight, out, rows, weight.outs, False, bias)
            else:
                operand, packed_rows = self._operand_rows(x, rows, weight.k)
                self._check(self.lib.akv_linear_packed(_ptr(operand), _ptr(weight.data), _ptr(out), _code(out), rows,
                                                       weight.outs, weight.k, weight.n_tiles, weight.k_tiles,
                                                       packed_rows, _ptr(bias), self._stream()), "linear")
            return
        rows, k = x.shape
        outs = weight.shape[0]
        self._dense(x, "x")
        self._dense(weight, "weight", None, (outs, k))
        self._dense(out, "out", None, (rows, outs))
        self._bias(bias, outs)
        self._check(self.lib.akv_linear_tiled(_ptr(x), _code(x), _ptr(weight), _code(weight), _ptr(out), _code(out),
                                              rows, outs, k, _ptr(bias), self._stream()), "linear")

    def _library_bias(self, bias: torch.Tensor) -> torch.Tensor:
        """The bias as the library's product wants it: bfloat16, made once per bias and kept (a bias read from a
        16-bit checkpoint is exact in bfloat16)."""
        known = self.__dict__.setdefault("_library_biases", {})
        key = bias.data_ptr()
        if key not in known or known[key][0] is not bias:
            known[key] = (bias, bias.to(torch.bfloat16))
        return known[key][1]

    # ---- decode steps: the residual sum and the norm inside the products -----------------------------------------
    FOLD_NORM_ROWS = 16             # steps of up to this many rows fold the residual sum and the norm into products
                                    # (measured from 1 to 16 rows at Qwen3-8B sizes: 5 to 14 us less per layer)
    FOLD_NORM_BYTES = 160 * 1024 - 832   # ... while the normed rows fit into a compute unit's LDS beside the scales
    fold_norms = True
    fold_rows_left = True           # ... the adding product leaving the rows times the next norm's weight, so that
                                    # the reading one only scales its sums (`linear_rowscaled`) instead of norming rows
    FOLD_MID_ROWS = 512             # ... and steps of up to this many, where the mid-size kernel takes the products:
    fold_mid = True                 # (a layer launches two norm kernels less: 5 us each and the gaps around them)

    def folds_norm(self, rows: int, hidden: int, dtype) -> bool:
        """Whether a step of `rows` rows may let a branch's last product add itself to the residual sum
        (`add_to_stream`) and the next product take the norm upon itself: up to 16 rows it norms the rows from the
        sums left there (`linear_scaled`); up to 512 it reads rows that the adding product left multiplied by the
        norm's weight and divides its results by the rows' root mean square (`linear_rowscaled`)."""
        if dtype != torch.bfloat16 or hidden % 8 != 0:
            return False
        if 0 < rows <= self.FOLD_NORM_ROWS:     # (a product that norms its rows itself keeps them in LDS)
            return self.fold_norms and (self.fold_rows_left or rows * hidden * 2 <= self.FOLD_NORM_BYTES)
        return self.fold_mid and rows <= self.FOLD_MID_ROWS

    def _reserve_exchange(self, n_tiles: int) -> None:
        """Called when a matrix is prepared: the memory through which two blocks of a decode product exchange the sums
        of a row tile whose parts of k they share (512 floats and a counter per row tile, and one tile more: a wave's
        pair of row tiles may begin at the last one; the counters are zero between launches).  One pair of buffers for
        all products - they follow each other on the stream."""
        n_tiles += 1
        if self._exchange_tiles < n_tiles:
            self._exchange_tiles = max(n_tiles, 4096)
            self._outgrown += [self._exchange_pieces, self._exchange_arrivals]
            self._exchange_pieces = torch.empty(self._exchange_tiles * 512, dtype=torch.float32, device=self.device)
            self._exchange_arrivals = torch.zeros(self._exchange_tiles, dtype=torch.int32, device=self.device)

    def _exchange(self, n_tiles: int):
        """The exchange buffers if they serve a matrix of `n_tiles` row tiles (they do for every prepared matrix; they
        are never replaced inside a step, whose recording may hold their addresses) - else the product keeps whole
        row tiles in a block."""
        if self._exchange_tiles < n_tiles + 1:
            return None, None
        return self._exchange_pieces, self._exchange_arrivals

    def decode_plan(self, weight, row_tiles_per_wave: int = 1, normed_rows: int = 0) -> dict:
        """How `linear_adds` / `linear_scaled` cut a product over this matrix into blocks (for tests and measurements)."""
        packed = weight.packed if isinstance(weight, GatedWeight) else weight
        out = (ctypes.c_int * 5)()
        may = 1 if self._exchange(packed.n_tiles)[0] is not None else 0
        self.lib.akv_linear_decode_plan(row_tiles_per_wave, packed.n_tiles, packed.k_tiles, packed.k, normed_rows, may, out)
        return dict(k_split=out[0], waves=out[1], blocks=out[2], straddles=bool(out[3]), work_kb=out[4])

    def adds_to_stream(self, rows: int, weight, dtype, gain=None) -> bool:
        if not isinstance(weight, PackedWeight) or not self.folds_norm(rows, weight.outs, dtype):
            return False
        if rows <= self.FOLD_NORM_ROWS:
            return True
        # many rows: the mid-size kernel, which must know the weight of the norm that follows
        return gain is not None and self._route("linear", weight.outs, weight.k, rows, weight.row_major is not None,
                                                torch.bfloat16) == "mid"

    def add_to_stream(self, x, weight: PackedWeight, stream, arena, bias=None, gain=None):
        """stream [rows, outs] (float32) += bfloat16(x W^T (+ bias)) in place; returns what the product left for the
        norm that follows (`StreamSums`): the rows' partial sums of squares, and in steps of more than 16 rows the
        new rows times `gain` as well."""
        from ..parts.base import StreamSums
        rows = x.shape[0]
        if rows <= self.FOLD_NORM_ROWS:
            sums = arena.take(((weight.outs + 15) // 16, 16), torch.float32)
            if gain is None or not self.fold_rows_left:
                self.linear_adds(x, weight, stream, sums, bias=bias)
                return StreamSums(sums)
            left = arena.take((rows, weight.outs), torch.bfloat16)
            self.linear_adds(x, weight, stream, sums, bias=bias, rows_out=left, gain=gain)
            return StreamSums(sums, rows=left, gain=gain)
        self._dense(x, "x", torch.bfloat16, (rows, weight.k))
        self._dense(stream, "stream", torch.float32, (rows, weight.outs))
        self._dense(gain, "norm weight", torch.float32, (weight.outs,))
        self._dense(weight.data, "packed weight", torch.bfloat16)
        self._bias(bias, weight.outs)
        bands = self.lib.akv_linear_mid_bands(rows, weight.n_tiles, weight.k_tiles)
        sums = arena.take((bands, (rows + 15) // 16 * 16), torch.float32)
        left = arena.take((rows, weight.outs), torch.bfloat16)
        self._mid(x, weight, left, rows, weight.outs, False, bias, adds=(stream, gain, sums))
        return StreamSums(sums, rows=left, gain=gain)

    def scales_rows_in_product(self, rows: int, weight, dtype, sums) -> bool:
        gated = isinstance(weight, GatedWeight)
        packed = weight.packed if gated else weight
        if not isinstance(packed, PackedWeight) or sums.rows is None or dtype != torch.bfloat16:
            return False
        if rows <= self.FOLD_NORM_ROWS:         # the decode products
            return self.fold_norms and rows > 0 and packed.k % 8 == 0 and tuple(sums.sums.shape) == ((packed.k + 15) // 16, 16)
        if rows > self.FOLD_MID_ROWS or sums.sums.shape[0] > self.lib.akv_linear_mid_most_groups(rows):
            return False
        if gated:
            return self._route("gated", weight.inter, packed.k, rows, weight.stacked is not None, dtype) == "mid"
        return self._route("linear", packed.outs, packed.k, rows, packed.row_major is not None, dtype) == "mid"

    def linear_rowscaled(self, x, sums, eps, weight, out, bias=None, row_tiles: int = 0) -> None:
        """out = (x W^T) with every row divided by sqrt(mean of squares + eps), plus `bias` (a `GatedWeight`: silu of
        the scaled gate times the scaled up): x [rows, k] are rows that `add_to_stream` left - the residual sum times
        the norm's weight -, sums [groups, rows rounded up to 16] the partial sums of squares of the residual rows."""
        gated = isinstance(weight, GatedWeight)
        packed = weight.packed if gated else weight
        rows = x.shape[0]
        outs = weight.inter if gated else packed.outs
        self._dense(x, "x", torch.bfloat16, (rows, packed.k))
        self._dense(out, "out", torch.bfloat16, (rows, outs))
        self._dense(packed.data, "packed weight", torch.bfloat16)
        if bias is not None and gated:
            raise KernelError("the gated product takes no bias")
        self._bias(bias, outs)
        if rows <= self.FOLD_NORM_ROWS:         # a decode step: sums per (16 values of a row, row), as `linear_adds` leaves them
            self._dense(sums, "sums", torch.float32, ((packed.k + 15) // 16, 16))
            pieces, arrivals = self._exchange(packed.n_tiles)
            self._check(self.lib.akv_linear_rowscaled(_ptr(x), _ptr(sums), (packed.k + 15) // 16, ctypes.c_float(eps),
                                                      _ptr(packed.data), _ptr(out), _ptr(pieces), _ptr(arrivals),
                                                      self._exchange_tiles if pieces is not None else 0, rows, outs,
                                                      packed.k, packed.n_tiles, packed.k_tiles, 1 if gated else 0,
                                                      row_tiles, _ptr(bias), self._stream()), "linear_rowscaled")
            return
        self._dense(sums, "sums", torch.float32, (sums.shape[0], (rows + 15) // 16 * 16))
        self._mid(x, packed, out, rows, outs, gated, bias, scaled=(sums, eps))

    def norms_rows_in_product(self, rows: int, weight, dtype) -> bool:
        packed = weight.packed if isinstance(weight, GatedWeight) else weight
        return (isinstance(packed, PackedWeight) and 0 < rows <= self.FOLD_NORM_ROWS and self.fold_norms
                and dtype == torch.bfloat16 and packed.k % 8 == 0 and rows * packed.k * 2 <= self.FOLD_NORM_BYTES)

    def linear_adds(self, x, weight: PackedWeight, stream, sums, bias=None, rows_out=None, gain=None) -> None:
        """stream [rows, outs] (float32) += bfloat16(x W^T (+ bias)), in place; sums [ceil(outs / 16), 16] (float32) receives
        per tile of 16 outputs and row the sum of squares of the new values; `rows_out` [rows, outs] bfloat16, if
        given, the new sum times `gain` [outs] (the weight of the norm that follows: what `linear_rowscaled` reads)."""
        rows = x.shape[0]
        if not isinstance(weight, PackedWeight) or rows > 16:
            raise KernelError("the product that adds to the residual sum takes a packed matrix and up to 16 rows")
        self._dense(x, "x", torch.bfloat16, (rows, weight.k))
        self._dense(stream, "stream", torch.float32, (rows, weight.outs))
        self._dense(sums, "sums", torch.float32, ((weight.outs + 15) // 16, 16))
        self._dense(weight.data, "packed weight", torch.bfloat16)
        pieces, arrivals = self._exchange(weight.n_tiles)
        if rows_out is not None:
            self._dense(rows_out, "rows_out", torch.bfloat16, (rows, weight.outs))
            self._dense(gain, "norm weight", torch.float32, (weight.outs,))
            self._check(self.lib.akv_linear_adds_rows(_ptr(x), _ptr(weight.data), _ptr(stream), _ptr(sums), _ptr(pieces),
                                                      _ptr(arrivals), self._exchange_tiles if pieces is not None else 0,
                                                      rows, weight.outs, weight.k, weight.n_tiles, weight.k_tiles,
                                                      _ptr(self._bias(bias, weight.outs)), _ptr(rows_out), _ptr(gain),
                                                      self._stream()), "linear_adds")
            return
        self._check(self.lib.akv_linear_adds(_ptr(x), _ptr(weight.data), _ptr(stream), _ptr(sums), _ptr(pieces),
                                             _ptr(arrivals), self._exchange_tiles if pieces is not None else 0,
                                             rows, weight.outs, weight.k, weight.n_tiles,
                                             weight.k_tiles, _ptr(self._bias(bias, weight.outs)), self._stream()),
                    "linear_adds")

    def linear_scaled(self, stream, sums, norm_weight, eps, weight, out, row_tiles: int = 0, bias=None) -> None:
        """out = norm(stream) W^T (a `GatedWeight`: silu(. Wgate^T) * (. Wup^T)) with the norm of `add_rmsnorm`
        (scaled, rounded, times the weight, rounded) applied to the float32 rows as they become operands; the rows'
        sums of squares are not formed but added up from `sums`, as `linear_adds` left them.  `row_tiles` forces the
        row tiles a wave of the plain product takes (1 or 2; for tests and measurements)."""
        gated = isinstance(weight, GatedWeight)
        packed = weight.packed if gated else weight
        rows, k = stream.shape
        if not isinstance(packed, PackedWeight) or rows > 16 or k != packed.k:
            raise KernelError("the product that norms its rows takes a packed matrix of the rows' width and up to 16 rows")
        self._dense(stream, "stream", torch.float32, (rows, k))
        self._dense(sums, "sums", torch.float32, ((k + 15) // 16, 16))
        self._dense(norm_weight, "norm weight", torch.float32, (k,))
        outs = weight.inter if gated else packed.outs
        self._dense(out, "out", torch.bfloat16, (rows, outs))
        self._dense(packed.data, "packed weight", torch.bfloat16)
        if bias is not None and gated:
            raise KernelError("the gated product takes no bias")
        self._bias(bias, outs)
        pieces, arrivals = self._exchange(packed.n_tiles)
        self._check(self.lib.akv_linear_scaled(_ptr(stream), _ptr(sums), (k + 15) // 16, _ptr(norm_weight),
                                               ctypes.c_float(eps), _ptr(packed.data), _ptr(out), _ptr(pieces),
                                               _ptr(arrivals), self._exchange_tiles if pieces is not None else 0,
                                               rows, outs, k, packed.n_tiles, packed.k_tiles,
                                               1 if gated else 0, row_tiles, _ptr(bias), self._stream()), "linear_scaled")

    STATIC_ROWS_ELEMENTS = 64 * 32768   # bfloat16 elements of the library's static device memory for repacked rows

    def linear_without_allocation(self, x, weight: PackedWeight, out) -> None:
        """out = x W^T for up to 64 bfloat16 rows through `akv_linear_packed_static`: the activations are repacked into
        static device memory of the library instead of a buffer of this kernel set, so neither this call nor anything
        under it allocates - for callers that must not (a graph being captured, a loop that may not touch the
        allocator).  Calls that overlap on one GPU share that memory and race; calls on one stream do not."""
        if not isinstance(weight, PackedWeight):
            raise KernelError("the product without allocation takes a packed bfloat16 matrix")
        rows = x.shape[0]
        self._dense(x, "x", torch.bfloat16, (rows, weight.k))
        self._dense(out, "out", None, (rows, weight.outs))
        self._dense(weight.data, "packed weight", torch.bfloat16)
        if rows > 64 or (rows + 15) // 16 * 16 * weight.k > self.STATIC_ROWS_ELEMENTS:
            raise KernelError(f"{rows} rows of {weight.k} do not fit the static memory of the product without allocation: "
                              f"at most 64 rows and {self.STATIC_ROWS_ELEMENTS} elements after rounding the rows up to 16")
        status = self.lib.akv_linear_packed_static(_ptr(x), _ptr(weight.data), _ptr(out), _code(out), rows, weight.outs,
                                                   weight.k, weight.n_tiles, weight.k_tiles, self._stream())
        if status == -3:
            raise KernelError("the product without allocation refused the sizes: they exceed its static memory")
        self._check(status, "linear_without_allocation")

    # The most rows whose norm the product's blocks compute for themselves.  Every block reads the rows again (24 KB a
    # row at 4,096 wide): measured at Qwen3-8B sizes, a step of one row gains 0.16 ms of 4.09, two rows lose 0.04 ms,
    # four lose 0.21 ms - so it is one.  (The kernel takes up to four.)
    NORM_IN_PRODUCT_ROWS = 1

    def norm_in_product(self, rows: int, weight, dtype) -> bool:
        """Whether `linear_after_norm` takes this product: a few bfloat16 rows, a packed matrix, rows that fit the
        block's LDS beside its sums."""
        packed = weight.packed if isinstance(weight, GatedWeight) else weight
        return (self.norm_in_products and 0 < rows <= self.NORM_IN_PRODUCT_ROWS and dtype == torch.bfloat16
                and isinstance(packed, PackedWeight) and packed.k % 8 == 0 and rows * packed.k * 2 <= 48 * 1024)

    def linear_after_norm(self, stream, delta, norm_weight, eps, stream_out, weight, out, bias=None):
        """out = norm(stream (+ delta)) W^T (a `GatedWeight`: silu(. Wgate^T) * (. Wup^T)) without a kernel for the
        norm: every block of the product adds, norms and rounds the few rows itself, as `add_rmsnorm` would, while its
        first weights are on their way.  stream [rows, k] float32 is not changed; stream_out [rows, k], another
        buffer, receives stream + delta."""
        gated = isinstance(weight, GatedWeight)
        packed = weight.packed if gated else weight
        rows, k = stream.shape
        if not self.norm_in_product(rows, weight, out.dtype):
            raise KernelError("this product does not take rows that are still to be normed")
        self._dense(stream, "stream", torch.float32, (rows, packed.k))
        self._dense(stream_out, "stream_out", torch.float32, (rows, k))
        if stream_out.data_ptr() == stream.data_ptr():
            raise KernelError("stream_out must be another buffer than stream")
        if delta is not None:
            self._dense(delta, "delta", torch.bfloat16, (rows, k))
        self._dense(norm_weight, "norm weight", torch.float32, (k,))
        outs = weight.inter if gated else packed.outs
        self._dense(out, "out", torch.bfloat16, (rows, outs))
        self._dense(packed.data, "packed weight", torch.bfloat16)
        self._check(self.lib.akv_linear_packed_normed(
            _ptr(stream), _ptr(delta), _ptr(norm_weight), ctypes.c_float(eps), _ptr(stream_out), _ptr(packed.data),
            _ptr(out), rows, outs, k, packed.n_tiles, packed.k_tiles, 1 if gated else 0,
            _ptr(self._bias(bias, outs) if not gated else None), self._stream()), "linear_after_norm")

    def prepare_gated_linear(self, gate: torch.Tensor, up: torch.Tensor):
        """The packing for `gated_linear`, or None where the two matrices have to stay a stacked product followed by
        `swiglu` (float32 weights, sizes the packed kernels do not take)."""
        if (gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16 and gate.shape == up.shape
                and gate.shape[1] % 8 == 0 and gate.shape[0] % 16 == 0):
            weight = GatedWeight(gate, up, keep_row_major=self.library_products_above is not None)
            self._products.setdefault(("gated", weight.inter, weight.k), weight)
            self._reserve_exchange(weight.packed.n_tiles)
            return weight
        return None

    def gated_scratch(self, weight: GatedWeight, rows: int, dtype: torch.dtype):
        """Shape of the buffer `gated_linear` wants for this many rows (the stacked product of the library path),
        or None."""
        wanted = (rows > 16 and dtype == torch.bfloat16
                  and self._route("gated", weight.inter, weight.k, rows, weight.stacked is not None, dtype) == "library")
        return (rows, 2 * weight.inter) if wanted else None

    def gated_linear(self, x, weight: GatedWeight, out, scratch=None):
        """out [rows, inter] = silu(x Wgate^T) * (x Wup^T): one kernel, from float32 accumulators; where the library
        takes the product, its stacked product into `scratch`, then the activation kernel."""
        rows = x.shape[0]
        packed = weight.packed
        self._dense(x, "x", torch.bfloat16, (rows, weight.k))
        self._dense(out, "out", None, (rows, weight.inter))
        self._dense(packed.data, "packed weight", torch.bfloat16)
        route = "own" if rows <= 16 else self._route("gated", weight.inter, weight.k, rows, weight.stacked is not None,
                                                     out.dtype)
        if route == "library":
            if scratch is None:
                raise KernelError(f"gated_linear of {rows} rows takes the library path and needs the scratch "
                                  "buffer that gated_scratch() describes")
            self._dense(scratch, "scratch", torch.bfloat16, (rows, 2 * weight.inter))
            torch.mm(x, weight.stacked.t(), out=scratch)
            self.swiglu(scratch, out)
        elif route == "mid":
            self._mid(x, packed, out, rows, weight.inter, True)
        else:
            operand, packed_rows = self._operand_rows(x, rows, weight.k)
            self._check(self.lib.akv_linear_packed_swiglu(_ptr(operand), _ptr(packed.data), _ptr(out), _code(out), rows,
                                                          weight.inter, weight.k, packed.n_tiles, packed.k_tiles,
                                                          packed_rows, self._stream()), "gated_linear")

    def swiglu(self, gate_up, out):
        tokens, inter = out.shape
        self._dense(gate_up, "gate_up", out.dtype, (tokens, 2 * inter))
        self._dense(out, "out")
        self._check(self.lib.akv_swiglu(_ptr(gate_up), _ptr(out), _code(out), ctypes.c_long(tokens), inter,
                                        self._stream()), "swiglu")

    # ---- position ----------------------------------------------------------------------------------------
    def rope_table(self, inv_freq, table):
        positions, half, two = table.shape
        self._dense(inv_freq, "inv_freq", torch.float32, (half,))
        self._dense(table, "table", torch.float32, (positions, half, 2))
        self._check(self.lib.akv_rope_table(_ptr(inv_freq), _ptr(table), positions, half, self._stream()), "rope_table")

    def rope(self, x, positions, table):
        tokens, heads, dim = x.shape
        self._dense(x, "x")
        self._dense(positions, "positions", torch.int32, (tokens,))
        self._dense(table, "table", torch.float32, (table.shape[0], dim // 2, 2))
        if dim % 2:
            raise KernelError("rotary head width must be even")
        self._check(self.lib.akv_rope(_ptr(x), _code(x), _ptr(positions), _ptr(table), ctypes.c_long(tokens), heads,
                                      dim, table.shape[0], self._stream()), "rope")

    # ---- cache -------------------------------------------------------------------------------------------
    def _pages(self, k_pages, v_pages, kv_heads, dim, dtype):
        self._dense(k_pages, "k_pages", dtype)
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != dim:
            raise KernelError(f"key pages must be [pages, {kv_heads}, page_size, {dim}], got {tuple(k_pages.shape)}")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
        self._dense(v_pages, "v_pages", dtype, (num_pages, kv_heads, dim, page_size))
        return num_pages, page_size

    def kv_write(self, k, v, slot_map, k_pages, v_pages):
        tokens, kv_heads, dim, k_stride = self._rows_view(k, "k")
        tv, hv, dv, v_stride = self._rows_view(v, "v")
        if (tv, hv, dv) != (tokens, kv_heads, dim) or v.dtype != k.dtype:
            raise KernelError("k and v must agree in shape and dtype")
        num_pages, page_size = self._pages(k_pages, v_pages, kv_heads, dim, k.dtype)
        self._dense(slot_map, "slot_map", torch.int32, (tokens,))
        self._check(self.lib.akv_kv_write(_ptr(k), ctypes.c_long(k_stride), _ptr(v), ctypes.c_long(v_stride),
                                          _ptr(slot_map), _ptr(k_pages), _ptr(v_pages), _code(k),
                                          ctypes.c_long(tokens), kv_heads, dim, page_size, ctypes.c_long(num_pages),
                                          self._stream()), "kv_write")

    def qk_norm_rope_write(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q_out,
                           q_heads, kv_heads, head_dim):
        tokens = qkv.shape[0]
        self._dense(qkv, "qkv", None, (tokens, (q_heads + 2 * kv_heads) * head_dim))
        self._dense(q_out, "q_out", qkv.dtype, (tokens, q_heads * head_dim))
        if (q_weight is None) != (k_weight is None):
            raise KernelError("q and k are normed together or not at all")
        if q_weight is not None:
            self._dense(q_weight, "q_weight", torch.float32, (head_dim,))
            self._dense(k_weight, "k_weight", torch.float32, (head_dim,))
        table_positions = 0
        if table is not None:
            self._dense(table, "table", torch.float32, (table.shape[0], head_dim // 2, 2))
            table_positions = table.shape[0]
        self._dense(positions, "positions", torch.int32, (tokens,))
        num_pages, page_size = self._pages(k_pages, v_pages, kv_heads, head_dim, qkv.dtype)
        if slot_map is not None:
            self._dense(slot_map, "slot_map", torch.int32, (tokens,))
        self._check(self.lib.akv_qk_norm_rope_write(
            _ptr(qkv), _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps), _ptr(table), table_positions,
            _ptr(positions), _ptr(slot_map), _ptr(k_pages), _ptr(v_pages), _ptr(q_out), _code(qkv),
            ctypes.c_long(tokens), q_heads, kv_heads, head_dim, page_size, ctypes.c_long(num_pages), self._stream()),
            "qk_norm_rope_write")

    def _attention_mfma_entry(self, head_dim: int):
        if head_dim not in self._attention_entry:
            path = ensure_attention(head_dim)
            try:
                lib = ctypes.CDLL(path)
            except OSError as error:
                raise KernelError(f"the attention library {path} could not be loaded: {error}") from error
            entry = getattr(lib, f"akv_attention_mfma_d{head_dim}")
            entry.restype = ctypes.c_int
            self._attention_entry[head_dim] = entry
        return self._attention_entry[head_dim]

    def _attention_pair_entry(self, head_dim: int):
        key = ("pair", head_dim)
        if key not in self._attention_entry:
            self._attention_mfma_entry(head_dim)            # (loads the head size's library)
            lib = ctypes.CDLL(ensure_attention(head_dim))
            entry = getattr(lib, f"akv_attention_pair_d{head_dim}")
            entry.restype = ctypes.c_int
            self._attention_entry[key] = entry
        return self._attention_entry[key]

    def _pair_fits(self, ctx, decodes, q_heads, kv_heads, head_dim, page_size, fresh) -> bool:
        """Whether a step's single tokens and prompt portions can go into one launch: the single tokens' kernel takes
        raw projections and cuts the keys on the device (at most 64 requests, some history beyond one segment), the
        portions are so short that their blocks of four narrow tiles do not fill the device, and no history of theirs
        is so long that its keys would be cut."""
        if not (self.pair_launch and fresh is not None and 0 < decodes <= 64 and head_dim % 64 == 0 and page_size >= 8
                and self.share_prompt_tiles and self.cut_keys_on_device and self.split_prompt_keys is not True
                and self.wide_prompt_tiles is not True):
            return False
        if max(ctx.host_seq_lens[:decodes]) <= self.decode_min_segment:
            return False
        if self._portion_blocks(ctx, decodes, q_heads, kv_heads) > self.compute_units:
            return False
        return not self._few_portion_blocks(ctx, decodes, q_heads, kv_heads)

    def _attention_pair(self, q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out,
                        page_size, num_pages, decodes, fresh):
        """Requests 0 .. decodes - 1 (single tokens, raw projections in `fresh`) and the prompt portions behind them in
        one launch of `akv_attention_pair`, then the single tokens' merge."""
        group = q_heads // kv_heads
        heads_per_tile = min(group, 16)
        head_groups = (group + heads_per_tile - 1) // heads_per_tile
        tokens_per_tile = 16 // heads_per_tile
        starts = ctx.host_q_start
        per_block = 4 * tokens_per_tile
        portion_tiles = sum((starts[r + 1] - starts[r] + per_block - 1) // per_block for r in range(decodes, ctx.num_seqs))
        # (the portions' blocks - four waves each - stand beside the single tokens' waves: together they are what one
        # round of the device holds, or the single tokens' last blocks wait for a second round)
        portion_waves = 4 * portion_tiles * kv_heads * head_groups
        waves = max(self.decode_wave_target // 2, self.decode_wave_target - portion_waves)
        plan, items_grid = self._decode_plan(ctx, 0, decodes, window, kv_heads * head_groups, waves)
        count = items_grid * kv_heads * head_groups * 16 * (head_dim + 4)
        arena = getattr(ctx, "arena", None)
        partial = (arena.take((count,), torch.float32) if arena is not None
                   else torch.empty(count, dtype=torch.float32, device=self.device))
        qkv, q_weight, k_weight, eps, table = fresh
        self._check(self._attention_pair_entry(head_dim)(
            _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(ctx.q_start), _ptr(ctx.seq_lens),
            _ptr(meta.block_table), _ptr(getattr(meta, "rows", None)), meta.width, q_heads, kv_heads, page_size,
            ctypes.c_long(num_pages), ctypes.c_float(scale), int(window) if window is not None else 0,
            0, decodes, heads_per_tile, head_groups, _ptr(partial), _ptr(plan), items_grid, _ptr(qkv), _ptr(q_weight),
            _ptr(k_weight), ctypes.c_float(eps), _ptr(table), table.shape[0] if table is not None else 0,
            decodes, ctx.num_seqs - decodes, portion_tiles, heads_per_tile, head_groups, tokens_per_tile,
            self._stream()), "attention")

    def _attention_mfma(self, q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out,
                        page_size, num_pages, seq_first, seq_count, nq, split, shared=False, fresh=None, single=None):
        """Requests seq_first .. seq_first + seq_count - 1 of the step on the MFMA kernel, in tiles of 16 * nq
        (token, head-of-group) columns; `split` cuts the keys over several waves whose partial results a second
        kernel merges; `single` (default: as `split`) says that each request brings one token (decode); `shared`
        (prompt portions, pages of 8 tokens and more) lets blocks of four waves, four tiles, fetch every key and
        value once into LDS; `fresh` (single tokens): (qkv, q_weight, k_weight, eps, table), the raw projections that
        the kernel norms, rotates and writes to the cache itself."""
        if single is None:
            single = split
        group = q_heads // kv_heads
        heads_per_tile = min(group, 16 * nq)
        head_groups = (group + heads_per_tile - 1) // heads_per_tile
        tokens_per_tile = (16 * nq) // heads_per_tile
        starts = ctx.host_q_start
        per_tile = tokens_per_tile * (4 if shared else 1)
        tiles = sum((starts[r + 1] - starts[r] + per_tile - 1) // per_tile
                    for r in range(seq_first, seq_first + seq_count))
        num_splits, seg_keys, partial, plan, items_grid = 1, 0, None, None, 0
        arena = getattr(ctx, "arena", None)
        take = lambda count: (arena.take((count,), torch.float32) if arena is not None
                              else torch.empty(count, dtype=torch.float32, device=self.device))
        if (split and single and self.cut_keys_on_device and seq_count <= 64
                and max(ctx.host_seq_lens[seq_first:seq_first + seq_count]) > self.decode_min_segment):
            # single tokens: their keys are cut on the device, from the lengths there (requests of 128 keys or
            # fewer are not cut: then the kernel without merge)
            plan, items_grid = self._decode_plan(ctx, seq_first, seq_count, window, kv_heads * head_groups)
            partial = take(items_grid * kv_heads * head_groups * 16 * nq * (head_dim + 4))
        elif split:
            longest = max(ctx.host_seq_lens[seq_first:seq_first + seq_count])
            pairs = tiles * kv_heads * head_groups
            num_splits = max(1, min((self.decode_wave_target + pairs - 1) // pairs,
                                    (longest + self.decode_min_segment - 1) // self.decode_min_segment,
                                    self.decode_max_splits))
            seg_keys = ((longest + num_splits - 1) // num_splits + 31) // 32 * 32
            num_splits = (longest + seg_keys - 1) // seg_keys
            if num_splits > 1:
                partial = take(tiles * kv_heads * head_groups * num_splits * 16 * nq * (head_dim + 4))
        qkv, q_weight, k_weight, eps, table = fresh if fresh is not None else (None, None, None, 0.0, None)
        self._check(self._attention_mfma_entry(head_dim)(
            _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(partial), _ptr(ctx.q_start), _ptr(ctx.seq_lens),
            _ptr(meta.block_table), _ptr(getattr(meta, "rows", None)), meta.width, seq_first, seq_count, tiles, nq,
            q_heads, kv_heads, heads_per_tile,
            head_groups, tokens_per_tile, page_size, ctypes.c_long(num_pages), ctypes.c_float(scale),
            int(window) if window is not None else 0, seg_keys, num_splits, 1 if single else 0, 1 if shared else 0,
            _ptr(qkv), _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps), _ptr(table),
            table.shape[0] if table is not None else 0, _ptr(plan), items_grid, self._stream()),
            "attention")

    PLAN_ENTRIES = 132          # ints of a plan before its items (4 per item)

    def _decode_plan(self, ctx, seq_first, seq_count, window, head_blocks, waves=None):
        """The cut of the keys of requests seq_first .. + seq_count - 1 (single tokens) into (request, segment) items:
        segments of one size for all requests - about `decode_wave_target` waves in all, no segment shorter than
        `decode_min_segment` unless it is a request's only one - worked out by a one-wave kernel from the lengths on
        the device.  The cut depends on the lengths alone, so the layers of a step share one plan: it is remembered on
        the step's context.  Returns the plan and the bound on the number of items that sizes grids and buffers."""
        items = max(1, (waves if waves is not None else self.decode_wave_target) // head_blocks)
        key = (seq_first, seq_count, int(window) if window is not None else 0, items, self.decode_min_segment)
        plans = getattr(ctx, "decode_plans", None)
        if plans is None:
            plans = {}
            try:
                ctx.decode_plans = plans
            except AttributeError:
                pass
        if key in plans:
            return plans[key]
        smallest = self.decode_min_segment
        items_grid = min(items + seq_count, sum((length + smallest - 1) // smallest
                                                for length in ctx.host_seq_lens[seq_first:seq_first + seq_count]))
        if items_grid > 65535:
            raise KernelError(f"{items_grid} segments of keys in one launch; the grid holds 65,535")
        # plans live in buffers of the kernel set (a step's arenas are handed on from layer to layer), one per plan
        # of a step; a step's plans are made before any later step's, on the same stream
        index = len(plans)
        while len(self._plan_buffers) <= index:
            self._plan_buffers.append(None)
        need = self.PLAN_ENTRIES + 4 * items_grid
        if self._plan_buffers[index] is None or self._plan_buffers[index].numel() < need:
            if torch.cuda.is_current_stream_capturing() and self._plan_buffers[index] is not None:
                raise KernelError("a recorded step needs a larger plan of its keys than the steps before it")
            self._outgrown.append(self._plan_buffers[index])       # (a recorded step may still point at it)
            self._plan_buffers[index] = torch.empty(max(need, self.PLAN_ENTRIES + 4 * 4096), dtype=torch.int32,
                                                    device=self.device)
        plan = self._plan_buffers[index]
        self._dense(ctx.seq_lens, "seq_lens", torch.int32, (ctx.num_seqs,))
        self._check(self.lib.akv_decode_plan(_ptr(ctx.seq_lens), seq_first, seq_count, key[2], items, smallest,
                                             items_grid, _ptr(plan), self._stream()), "decode_plan")
        plans[key] = (plan, items_grid)
        return plans[key]

    def _few_portion_blocks(self, ctx, first, q_heads, kv_heads) -> bool:
        """Whether the prompt portions of the step are so short, and their histories so long, that blocks of four
        tiles would leave most compute units idle while each walks thousands of keys: then a wave takes a tile and a
        segment of the keys, as in decoding.  The histories are those of the portions' own requests (in a recorded
        step a bound on them), not of the single tokens beside them.  Measured at Qwen3-8B sizes, blocks of four tiles
        against cut keys:
        128 tokens after 4,096: 114 / 63 us; 64 after 8,192: 221 / 65; 32 after 16,384: 437 / 70; but 256 after
        2,048: 67 / 77, 128 after 1,024: 37 / 41, 512 after 4,096: 128 / 195."""
        return (4 * self._portion_blocks(ctx, first, q_heads, kv_heads) <= self.compute_units
                and max(ctx.host_seq_lens[first:ctx.num_seqs]) > 2048)

    def _portion_blocks(self, ctx, first, q_heads, kv_heads) -> int:
        """How many blocks of four tiles of 16 columns the step's prompt portions make."""
        group = q_heads // kv_heads
        heads_per_tile = min(group, 16)
        per_block = 4 * (16 // heads_per_tile)
        starts = ctx.host_q_start
        blocks = sum((starts[r + 1] - starts[r] + per_block - 1) // per_block for r in range(first, ctx.num_seqs))
        return blocks * kv_heads * ((group + heads_per_tile - 1) // heads_per_tile)

    def _wide_shared_tiles(self, ctx, first, q_heads, kv_heads) -> bool:
        """Whether the prompt portions of the step go to blocks of 4 x 32 columns rather than 4 x 16.  The wide
        blocks do a step of 32 keys for twice the columns with the same loads and bookkeeping (a fifth to a quarter
        faster where they fill the device), but there are half as many of them, and two per compute unit instead of
        three: they are taken when there are two or more per compute unit and the keys are many (measured on
        prompts of 512 to 8,192 tokens after histories of 0 to 15,360)."""
        group = q_heads // kv_heads
        heads_per_tile = min(group, 32)
        per_block = 4 * (32 // heads_per_tile)
        starts = ctx.host_q_start
        blocks = sum((starts[r + 1] - starts[r] + per_block - 1) // per_block for r in range(first, ctx.num_seqs))
        blocks *= kv_heads * ((group + heads_per_tile - 1) // heads_per_tile)
        units = self.compute_units
        return blocks >= 2 * units and (max(ctx.host_seq_lens[first:ctx.num_seqs]) >= 4096 or 2 * blocks >= 5 * units)

    def _matrix_core_attention(self, dtype, page_size) -> bool:
        fits = page_size >= 4 and page_size & (page_size - 1) == 0
        if dtype == torch.bfloat16 and not fits and not self.one_wave_per_head:
            self._warn_once(("page", page_size), f"cache pages of {page_size} tokens: the matrix-core attention takes pages of "
                            "4 tokens or more whose size is a power of two, so bfloat16 attention runs in the plain kernel, "
                            "one wave per token and head (correct, and many times slower)")
        return dtype == torch.bfloat16 and fits and not self.one_wave_per_head

    def _warn_once(self, key, message: str) -> None:
        """A kernel choice that keeps results right and costs much speed is said once, not silently made."""
        told = self.__dict__.setdefault("_told", set())
        if key not in told:
            told.add(key)
            import warnings
            warnings.warn(message, RuntimeWarning, stacklevel=3)

    def encode_and_attend(self, qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q, ctx,
                          meta, q_heads, kv_heads, head_dim, scale, window, out):
        """`qk_norm_rope_write` followed by `attention`, as one call: out[tokens, q_heads * head_dim] from the raw
        stacked projections qkv.  `slot_map` must name, for every token, the slot that the request's block table
        names for the token's position.  `q` is where encoded queries are kept between the two kernels.
        The requests that bring a single token (the first `ctx.num_decode_seqs`; their tokens are the step's first
        rows) need no kernel of their own for the first half where the attention kernel takes raw projections:
        it norms and rotates their queries and new keys in registers and writes the new keys and values itself."""
        tokens = qkv.shape[0]
        decodes = ctx.num_decode_seqs
        fresh = (self.fresh_decode_tokens and decodes > 0 and slot_map is not None and head_dim % 64 == 0
                 and self._matrix_core_attention(qkv.dtype, k_pages.shape[2] if k_pages.dim() == 4 else 0))
        if not fresh:
            self.qk_norm_rope_write(qkv, q_weight, k_weight, eps, table, positions, slot_map, k_pages, v_pages, q,
                                    q_heads, kv_heads, head_dim)
            self.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out)
            return
        if ctx.host_q_start[decodes] != decodes:
            raise KernelError("the single tokens of a step must be its first rows")
        self._dense(qkv, "qkv", torch.bfloat16, (tokens, (q_heads + 2 * kv_heads) * head_dim))
        if (q_weight is None) != (k_weight is None):
            raise KernelError("q and k are normed together or not at all")
        if q_weight is not None:
            self._dense(q_weight, "q_weight", torch.float32, (head_dim,))
            self._dense(k_weight, "k_weight", torch.float32, (head_dim,))
        if table is not None:
            self._dense(table, "table", torch.float32, (table.shape[0], head_dim // 2, 2))
        encode_portions = None
        if decodes < tokens:    # prompt portions: the kernel of the first half, on their rows alone
            encode_portions = lambda: self.qk_norm_rope_write(
                qkv[decodes:], q_weight, k_weight, eps, table, positions[decodes:], slot_map[decodes:], k_pages,
                v_pages, q[decodes:], q_heads, kv_heads, head_dim)
        self.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out,
                       fresh=(qkv, q_weight, k_weight, float(eps), table), encode_portions=encode_portions)

    def _fork(self):
        """A second stream that starts where the current one is (default priority, made once).  What is launched on
        it runs beside what the current stream is given next; `_join` makes the current stream wait for it.  Inside a
        recording the two become branches of the graph."""
        if self._beside_stream is None:
            self._beside_stream = torch.cuda.Stream(self.device)
        forked = torch.cuda.Event()
        forked.record(torch.cuda.current_stream(self.device))
        self._beside_stream.wait_event(forked)
        return self._beside_stream

    def _join(self, beside) -> None:
        joined = torch.cuda.Event()
        joined.record(beside)
        torch.cuda.current_stream(self.device).wait_event(joined)

    def attention(self, q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out, fresh=None,
                  encode_portions=None):
        """`fresh` and `encode_portions` are `encode_and_attend`'s: the raw projections of the step and what encodes
        them, and the launch that encodes the prompt portions' rows (it must precede the portions' attention and
        nothing else).
        A step of single tokens and short prompt portions: the two kinds read and write different requests' pages
        and different rows of `q` and `out`, and neither fills the device - the single tokens' keys stream from
        memory, the portions' few blocks (no more than there are compute units) wait for one load after the other.
        Where the two kernels can share a grid (`_pair_fits`) they are ONE launch, the portions' blocks first
        (`akv_attention_pair`); otherwise the portions' launches go to a second stream and the two run beside each
        other.  (Measured in a recorded step of 120 prompt tokens beside 8 x 8,192: 6.5 + 27 + 48 + 5 us one after
        the other; on two streams 66 us beside each other and about 15 us for the two waits between the streams.)"""
        tokens = q.shape[0]
        self._dense(q, "q", None, (tokens, q_heads * head_dim))
        self._dense(out, "out", q.dtype, (tokens, q_heads * head_dim))
        num_pages, page_size = self._pages(k_pages, v_pages, kv_heads, head_dim, q.dtype)
        rows = getattr(meta, "rows", None)
        if rows is None:    # a table of the step's own: row r is request r's
            self._dense(meta.block_table, "block_table", torch.int32, (ctx.num_seqs, meta.width))
        else:               # the persistent table: request r's pages are row rows[r] (its slot)
            self._dense(rows, "table rows", torch.int32, (ctx.num_seqs,))
            self._dense(meta.block_table, "block_table", torch.int32, (meta.block_table.shape[0], meta.width))
            if max(ctx.host_seq_slots) >= meta.block_table.shape[0] or min(ctx.host_seq_slots) < 0:
                raise KernelError("a request's slot lies outside the block table")
        if ctx.max_seq_len > meta.width * page_size:
            raise KernelError(f"a request of {ctx.max_seq_len} tokens does not fit a block table of {meta.width} pages")
        if fresh is not None and not self._matrix_core_attention(q.dtype, page_size):
            raise KernelError("raw projections are taken by the matrix-core attention alone")
        if self._matrix_core_attention(q.dtype, page_size):
            self._dense(ctx.q_start, "q_start", torch.int32, (ctx.num_seqs + 1,))
            self._dense(ctx.seq_lens, "seq_lens", torch.int32, (ctx.num_seqs,))
            if ctx.host_q_start[ctx.num_seqs] != tokens or len(ctx.host_seq_lens) != ctx.num_seqs:
                raise KernelError("the step's request boundaries do not match its tokens")
            common = (q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, head_dim, scale, window, out, page_size,
                      num_pages)
            decodes = ctx.num_decode_seqs

            def portions():
                if encode_portions is not None:
                    encode_portions()
                shared = page_size >= 8 and self.share_prompt_tiles
                nq = 2 if head_dim <= 128 else 1
                cut = self.split_prompt_keys
                if cut is None:
                    cut = self._few_portion_blocks(ctx, decodes, q_heads, kv_heads)
                if cut:     # short portions after long histories: too few blocks to fill the device, so the keys are cut
                    self._attention_mfma(*common, decodes, ctx.num_seqs - decodes, nq, True, single=False)
                    return
                if shared and nq == 2:
                    wide = self.wide_prompt_tiles
                    if wide is None:
                        wide = self._wide_shared_tiles(ctx, decodes, q_heads, kv_heads)
                    nq = 2 if wide else 1
                self._attention_mfma(*common, decodes, ctx.num_seqs - decodes, nq, False, shared=shared)

            if ctx.num_seqs > decodes and self._pair_fits(ctx, decodes, q_heads, kv_heads, head_dim, page_size, fresh):
                if encode_portions is not None:
                    encode_portions()
                self._attention_pair(*common, decodes, fresh)
                return
            beside = None
            if ctx.num_seqs > decodes:
                if (decodes > 0 and self.portions_beside_single_tokens
                        and self._portion_blocks(ctx, decodes, q_heads, kv_heads) <= self.compute_units):
                    beside = self._fork()
                    with torch.cuda.stream(beside):
                        portions()
                elif encode_portions is not None:
                    encode_portions()
                    encode_portions = None
            # single tokens against long histories: one small tile each, keys split over waves; 64 requests a launch
            for first in range(0, decodes, 64):
                self._attention_mfma(*common, first, min(64, decodes - first), 1, True, fresh=fresh)
            if beside is not None:
                self._join(beside)
            elif ctx.num_seqs > decodes:
                portions()
            return
        if encode_portions is not None:
            encode_portions()
        self._dense(ctx.seq_of_token, "seq_of_token", torch.int32, (tokens,))
        self._dense(ctx.positions, "positions", torch.int32, (tokens,))
        self._check(self.lib.akv_attention_rows(
            _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(ctx.seq_of_token), _ptr(ctx.positions),
            _ptr(meta.block_table), _ptr(rows), meta.width, _ptr(out), _code(q), ctypes.c_long(tokens), q_heads, kv_heads,
            head_dim, page_size, ctypes.c_long(num_pages), ctypes.c_float(scale),
            int(window) if window is not None else 0, self._stream()), "attention")

    # ---- sampling ----------------------------------------------------------------------------------------
    # A row of logits is cut over several blocks where the rows are few (one block on one compute unit takes 18 us
    # for 151,936 logits): enough parts for some 256 blocks, each of at least 2,048 logits.
    SAMPLE_PART_ROWS = 1024         # rows the parts' workspace serves; more rows have a block each anyway
    sample_in_parts = True

    def _sample_parts(self, rows: int, vocab: int) -> int:
        if not self.sample_in_parts or rows > self.SAMPLE_PART_ROWS:
            return 1
        parts = min(64, max(1, 256 // rows), vocab // 2048)
        if parts < 2:
            return 1
        if self._sample_workspace is None:
            if torch.cuda.is_current_stream_capturing():
                return 1
            self._sample_workspace = (torch.empty(self.SAMPLE_PART_ROWS * 64, dtype=torch.float32, device=self.device),
                                      torch.empty(self.SAMPLE_PART_ROWS * 64, dtype=torch.int32, device=self.device),
                                      torch.zeros(self.SAMPLE_PART_ROWS, dtype=torch.int32, device=self.device))
        return parts

    def sample(self, logits, temperature, seeds, draws, out):
        rows, vocab = logits.shape
        self._dense(logits, "logits", torch.float32)
        self._dense(out, "out", torch.int32, (rows,))
        if temperature is not None:
            self._dense(temperature, "temperature", torch.float32, (rows,))
            self._dense(seeds, "seeds", torch.int64, (rows,))
            self._dense(draws, "draws", torch.int32, (rows,))
        parts = self._sample_parts(rows, vocab)
        if parts > 1:
            values, ids, arrivals = self._sample_workspace
            self._check(self.lib.akv_sample_parts(_ptr(logits), _ptr(temperature), _ptr(seeds), _ptr(draws), None, None, None,
                                                  None, _ptr(out), rows, vocab, parts, _ptr(values), _ptr(ids),
                                                  _ptr(arrivals), self._stream()), "sample")
            return
        self._check(self.lib.akv_sample(_ptr(logits), _ptr(temperature), _ptr(seeds), _ptr(draws), _ptr(out), rows,
                                        vocab, self._stream()), "sample")

    def sample_slots(self, logits, ctx, out):
        """The next token of every wanted row of the step `ctx`, chosen with the sampling state that the row's request
        keeps in its slot (temperature, seed, draws so far); the chosen token and the new draw count are left there."""
        rows, vocab = logits.shape
        self._dense(logits, "logits", torch.float32)
        self._dense(out, "out", torch.int32, (rows,))
        self._dense(ctx.logit_rows, "logit_rows", torch.int32, (rows,))
        self._dense(ctx.seq_of_token, "seq_of_token", torch.int32, (ctx.num_tokens,))
        self._dense(ctx.seq_slots, "seq_slots", torch.int32, (ctx.num_seqs,))
        self._dense(ctx.slot_words, "slot_words", torch.int32)
        if max(ctx.host_seq_slots) >= ctx.slot_words.shape[0]:
            raise KernelError("a request's slot lies outside the slot words")
        parts = self._sample_parts(rows, vocab)
        if parts > 1:
            values, ids, arrivals = self._sample_workspace
            self._check(self.lib.akv_sample_parts(_ptr(logits), None, None, None, _ptr(ctx.logit_rows), _ptr(ctx.seq_of_token),
                                                  _ptr(ctx.seq_slots), _ptr(ctx.slot_words), _ptr(out), rows, vocab, parts,
                                                  _ptr(values), _ptr(ids), _ptr(arrivals), self._stream()), "sample_slots")
            return
        self._check(self.lib.akv_sample_slots(_ptr(logits), _ptr(ctx.logit_rows), _ptr(ctx.seq_of_token),
                                              _ptr(ctx.seq_slots), _ptr(ctx.slot_words), _ptr(out), rows, vocab,
                                              self._stream()), "sample_slots")

    def argmax(self, logits, out):
        self.sample(logits, None, None, None, out)
