"""One checked Python wrapper per HIP kernel.

Each wrapper verifies on the host what the kernel and its grid assume (device, dtype,
contiguity, shapes) and only then launches on torch's current stream.  Nothing here
computes with torch operators: if a library is missing the call raises.
"""

import functools
import math

import torch

from atomserve_amd.kernels.lib import KernelError, call, entry

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
_DT = {F32: 0, BF16: 1}


def _stream() -> int:
    """The raw handle of torch's current stream on the current device (an eager step makes some
    hundred launches, so this asks the binding directly instead of building a Stream object)."""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def _check(t, name, dtype=None, shape=None):
    """Runs before every launch, several times: written for the case that all is well."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name} must be a tensor on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype is not dtype and (isinstance(dtype, torch.dtype) or t.dtype not in dtype):
        raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
    if shape is not None:
        have = t.shape
        good = len(have) == len(shape)
        if good:
            for d, s in zip(have, shape):
                if s is not None and d != s:
                    good = False
                    break
        if not good:
            raise KernelError(f"{name} has shape {tuple(have)}, expected {tuple(shape)}")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ---- weights in the order in which a wave reads them -------------------------------------------
#
# The few-rows and tile products stream a weight matrix once per step.  `Streamed(w)` holds a bf16
# matrix [R, K] (R % 16 == 0, K % 64 == 0) a second time, its 16-byte pieces lying as a wave of those
# kernels takes them; the products that are handed the `Streamed` read that copy (every load
# instruction 1 KB in one piece, marked as not to be kept: 7 per cent less time for the 144 products of
# a decode step at Qwen3-8B sizes), the library's products and everything else read the rows.  The
# owner of the matrix (a part, the decoder for its head) owns the `Streamed` and with it the copy's
# memory; whoever changes the rows in place afterwards calls `refresh()`.


class Streamed:
    """A weight matrix as the products of this module read it: `rows`, the tensor [R, K] itself, and
    `wave`, its copy in wave order, or None where the dtype or the sizes do not allow one or the owner
    asked for none (`copy=False`: the copy's bytes are saved, decode steps stream the rows)."""

    __slots__ = ("rows", "wave")

    def __init__(self, rows, copy: bool = True):
        self.rows, self.wave = rows, None
        if copy:
            self.refresh()

    @staticmethod
    def possible(w) -> bool:
        return w.dtype == BF16 and w.dim() == 2 and w.is_cuda and w.is_contiguous() and w.shape[0] % 16 == 0 and w.shape[1] % 64 == 0

    def refresh(self):
        """Makes the copy (anew) from the rows as they are now; returns it, None where there can be none."""
        if not self.possible(self.rows):
            self.wave = None
            return None
        if self.wave is None:
            self.wave = torch.empty_like(self.rows)
        call("as_wave_order", _ptr(self.rows), _ptr(self.wave), self.rows.shape[0], self.rows.shape[1], _stream())
        return self.wave

    @property
    def wave_bytes(self) -> int:
        return 0 if self.wave is None else self.wave.numel() * self.wave.element_size()


def _rows(w):
    """The matrix itself of what a product was handed as its weights (a tensor, or a `Streamed`)."""
    return w.rows if isinstance(w, Streamed) else w


def _wave_ptr(w) -> int:
    """The address of the copy in wave order of a product's weights, 0 if they have none."""
    if isinstance(w, Streamed) and w.wave is not None:
        return w.wave.data_ptr()
    return 0


def embed_gather(table, ids, out, scale: float = 1.0) -> None:
    """out[t] = scale * table[ids[t]] as fp32.  table [V, h] fp32|bf16, ids [T] int32, out [T, h] fp32."""
    _check(table, "table", (F32, BF16), (None, None))
    vocab, width = table.shape
    _check(ids, "ids", I32, (None,))
    _check(out, "out", F32, (ids.shape[0], width))
    call("as_embed_gather", _ptr(table), _DT[table.dtype], _ptr(ids), _ptr(out), ids.shape[0], width, vocab,
         float(scale), _stream())  # fmt: skip


def logits_finish(logits, scale: float = 1.0, softcap: float = 0.0) -> None:
    """logits = softcap * tanh(scale * logits / softcap) in place (softcap 0: the scale alone); fp32."""
    _check(logits, "logits", F32)
    if softcap < 0:
        raise KernelError("a soft cap of logits is positive, or 0 for none")
    call("as_logits_finish", _ptr(logits), logits.numel(), float(scale), float(softcap), _stream())


def rmsnorm(x, weight, eps, out, delta=None, rows=None, update_x=True, split_sums=None) -> None:
    """out[r] = norm(x[s] + delta[s]) * weight with s = rows[r] (or r); x fp32 [T, n] gets the
    sum written back when `delta` is given and `update_x`.  out, delta: fp32|bf16.
    split_sums: instead of `delta`, the fp32 partial sums [splits, T, n] of the product that makes it
    (`gemm_split`); they are added up and rounded to out's dtype as the product would have been."""
    _check(x, "x", F32, (None, None))
    T, n = x.shape
    _check(weight, "weight", (F32, BF16), (n,))
    n_out = T
    if rows is not None:
        _check(rows, "rows", I32, (None,))
        n_out = rows.shape[0]
    _check(out, "out", (F32, BF16), (n_out, n))
    if delta is not None:
        _check(delta, "delta", out.dtype, (T, n))
    if out.dtype == F32 and weight.dtype != F32:
        raise KernelError("fp32 norm needs an fp32 weight")
    if split_sums is not None:
        if delta is not None:
            raise KernelError("a pending sum comes as one tensor or as partial sums, not both")
        _check(split_sums, "split_sums", F32, (None, T, n))
        call("as_rmsnorm_split", _ptr(x), _ptr(split_sums), split_sums.shape[0], T, _ptr(rows), _ptr(weight),
             _DT[weight.dtype], float(eps), _ptr(out), _DT[out.dtype], n_out, n, int(bool(update_x)), _stream())  # fmt: skip
        return
    call("as_rmsnorm", _ptr(x), _ptr(delta), _ptr(rows), _ptr(weight), _DT[weight.dtype], float(eps), _ptr(out),
         _DT[out.dtype], n_out, n, int(bool(update_x)), _stream())  # fmt: skip


def rope_table(positions, inv_freq, out, magnitude: float = 1.0) -> None:
    """out[t, i] = magnitude * (cos, sin)(positions[t] * inv_freq[i]); inv_freq fp64 [R/2], out fp32 [T, R/2, 2]."""
    _check(positions, "positions", I32, (None,))
    _check(inv_freq, "inv_freq", torch.float64, (None,))
    _check(out, "out", F32, (positions.shape[0], inv_freq.shape[0], 2))
    if magnitude == 1.0:
        call("as_rope_table", _ptr(positions), _ptr(inv_freq), _ptr(out), positions.shape[0], inv_freq.shape[0], _stream())
    else:
        call("as_rope_table_scaled", _ptr(positions), _ptr(inv_freq), _ptr(out), positions.shape[0], inv_freq.shape[0],
             float(magnitude), _stream())  # fmt: skip


def qk_norm_rope_store(qkv, q_weight, k_weight, cos_sin, slots, q_out, k_pages, v_pages, num_heads,
                       num_kv_heads, eps, store_kv=True) -> None:  # fmt: skip
    """Per-head norm (if weights are given), rotation (if `cos_sin` is given) and the cache store.

    qkv [T, H + 2 KV, D]; q_out [T, H, D]; k_pages [num_pages, KV, block_size, D], v_pages
    [num_pages, KV, D, block_size] (values transposed within a page); slots [T] int32
    (page * block_size + offset, or -1 for a token whose keys are not stored)."""
    _check(qkv, "qkv", (F32, BF16), (None, num_heads + 2 * num_kv_heads, None))
    T, _, D = qkv.shape
    _check(q_out, "q_out", qkv.dtype, (T, num_heads, D))
    R = 0
    if cos_sin is not None:
        _check(cos_sin, "cos_sin", F32, (T, None, 2))
        R = 2 * cos_sin.shape[1]
        if R > D:
            raise KernelError(f"rotary width {R} exceeds head width {D}")
    w_dtype = qkv.dtype
    if q_weight is not None:
        _check(q_weight, "q_weight", (F32, BF16), (D,))
        _check(k_weight, "k_weight", q_weight.dtype, (D,))
        w_dtype = q_weight.dtype
        if qkv.dtype == F32 and w_dtype != F32:
            raise KernelError("fp32 q/k norm needs fp32 weights")
    elif k_weight is not None:
        raise KernelError("q and k norm weights come together")
    block_size = 1
    if store_kv:
        _check(slots, "slots", I32, (T,))
        _check(k_pages, "k_pages", qkv.dtype, (None, num_kv_heads, None, D))
        block_size = k_pages.shape[2]
        _check(v_pages, "v_pages", qkv.dtype, (k_pages.shape[0], num_kv_heads, D, block_size))
    call("as_qk_norm_rope_store", _ptr(qkv), _DT[qkv.dtype], _ptr(q_weight), _ptr(k_weight), _DT[w_dtype],
         _ptr(cos_sin), _ptr(slots) if store_kv else 0, _ptr(q_out), _ptr(k_pages) if store_kv else 0,
         _ptr(v_pages) if store_kv else 0, T, num_heads, num_kv_heads, D, R, float(eps), block_size,
         int(bool(store_kv)), _stream())  # fmt: skip


def silu_mul(gate_up, out) -> None:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _check(gate_up, "gate_up", (F32, BF16), (None, None))
    T, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("gate_up needs an even width")
    _check(out, "out", gate_up.dtype, (T, two_i // 2))
    call("as_silu_mul", _ptr(gate_up), _ptr(out), _DT[gate_up.dtype], T, two_i // 2, _stream())


SINGLE_QUERY_MAX_HEAD_DIM = 256


def attn_single_query(q, k_pages, v_pages, items, positions, tok_row, block_tables, out, scale, window,
                      max_context, part_size=None, force_generic=False) -> None:  # fmt: skip
    """Attention of single query tokens over the paged cache.  bfloat16 with head widths in steps
    of 32 and pages of a multiple of 16 tokens runs on the matrix cores (a group of more than 16 query
    heads, or of wide heads that overfill a workgroup's LDS, as several equal groups that read the same kv
    head); everything else (and all of fp32) on the general kernel.

    q, out [T, H, D]; items [N] int32: the tokens (rows of q) to process, None for all of them in
    order; positions, tok_row [T] int32 (tok_row None: token t belongs to row t, a decode step);
    block_tables [R, W] int32; max_context: host bound on positions[items] + 1."""
    _check(q, "q", (F32, BF16), (None, None, None))
    T, H, D = q.shape
    _check(out, "out", q.dtype, (T, H, D))
    _check(k_pages, "k_pages", q.dtype, (None, None, None, D))
    _, KV, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q.dtype, (k_pages.shape[0], KV, D, bs))
    if items is not None:
        _check(items, "items", I32, (None,))
    _check(positions, "positions", I32, (T,))
    if tok_row is not None:
        _check(tok_row, "tok_row", I32, (T,))
    _check(block_tables, "block_tables", I32, (None, None))
    if tok_row is None and block_tables.shape[0] < T:
        raise KernelError(f"attention: {T} tokens that are their own rows need as many block tables")
    N = T if items is None else items.shape[0]
    if N == 0:
        return
    chunk = 4 if q.dtype == F32 else 8
    if H % KV or D % chunk or D > SINGLE_QUERY_MAX_HEAD_DIM:
        raise KernelError(f"attention: unsupported heads {H}/{KV} or head width {D} "
                          f"(needs a multiple of {chunk}, at most {SINGLE_QUERY_MAX_HEAD_DIM})")  # fmt: skip
    if max_context > block_tables.shape[1] * bs:
        raise KernelError("attention: block tables are shorter than the longest context")
    G = H // KV
    # a group of more query heads than the matrix-core kernel's workgroup takes is cut into equal smaller ones
    share = next((G // g for g in range(min(G, 16), 0, -1) if G % g == 0 and _decode_mfma_fits(D, g)), 0)
    mfma = q.dtype == BF16 and D % 32 == 0 and bs % 16 == 0 and share > 0 and not force_generic
    if mfma and share > 1:
        part_size, P, part_m, part_l, part_acc = _partitions(N, H, KV * share, D, max_context, window, True, part_size, q.device)
        call("as_attn_decode_mfma_shared", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(items), N, _ptr(positions),
             _ptr(tok_row), _ptr(block_tables), block_tables.shape[1], _ptr(out), _ptr(part_m), _ptr(part_l),
             _ptr(part_acc), H, KV * share, D, bs, float(scale), int(window), part_size, P, share, _stream())  # fmt: skip
        return
    part_size, P, part_m, part_l, part_acc = _partitions(N, H, KV, D, max_context, window, mfma, part_size, q.device)
    if mfma:
        call("as_attn_decode_mfma", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(items), N, _ptr(positions),
             _ptr(tok_row), _ptr(block_tables), block_tables.shape[1], _ptr(out), _ptr(part_m), _ptr(part_l),
             _ptr(part_acc), H, KV, D, bs, float(scale), int(window), part_size, P, _stream())  # fmt: skip
        return
    call("as_attn_single_query", _ptr(q), _ptr(k_pages), _ptr(v_pages), _DT[q.dtype], _ptr(items), N,
         _ptr(positions), _ptr(tok_row), _ptr(block_tables), block_tables.shape[1], _ptr(out), _ptr(part_m),
         _ptr(part_l), _ptr(part_acc), H, KV, D, bs, float(scale), int(window), part_size, P, _stream())  # fmt: skip


DECODE_MFMA_MAX_LDS = 64 << 10  # what a workgroup may ask for without raising the kernel's limit


def compute_units() -> int:
    """Compute units of the current GPU (256 on an MI355X); grids and the fitted costs below scale with it."""
    global _compute_units
    if _compute_units is None:
        _compute_units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return _compute_units


_compute_units = None


def _decode_mfma_fits(head_dim: int, group: int) -> bool:
    """Whether the matrix-core decode kernel's workgroup (queries of a group and four partial outputs
    in LDS) stays within the LDS a kernel gets unasked; wide heads in large groups do not."""
    return 4 * (128 + 4 * head_dim * group) + 1024 <= DECODE_MFMA_MAX_LDS


def attn_fill_groups() -> int:
    """(token, kv head) pairs from which on whole contexts beat partitions and their merge: one and a
    half per compute unit (measured on 256)."""
    return compute_units() * 3 // 2


MFMA_PARTITIONS = (128, 256, 512, 1024, 2048)  # keys per workgroup of the matrix-core decode kernel


def _partition_cost(groups: int, span: int, part: int) -> float:
    """Microseconds, roughly, of the decode attention and its merge when `groups` (token, kv head) pairs
    cut `span` keys into partitions of `part`: a workgroup costs 4 us and 25 ns a key, two of them run
    on a compute unit at a time, and the merge 0.6 us a partition.  Fitted to the kernel's times at 1
    to 32 requests of 500 to 33,000 keys (heads of 128, 8 kv heads, 256 compute units); what it picks
    is within 2 per cent of the best partition size on average there, where one size for all was 8 per
    cent off."""
    parts = math.ceil(span / part)
    return (4.0 + 0.025 * min(part, span)) * max(1.0, groups * parts / (2 * compute_units())) + 0.6 * parts


def _partitions(N, H, KV, D, max_context, window, mfma, part_size, device):
    """How the keys of N single queries are cut for the split-KV kernels, and the buffers of the
    partial results: (part_size, P, part_m, part_l, part_acc), the buffers None when P == 1."""
    span = min(max_context, window) if window > 0 else max_context
    G = H // KV
    if part_size is None:
        # Enough partitions to occupy the GPU when few tokens are in the batch, few enough that
        # the merge stays small; boundaries are multiples of part_size in absolute position.
        if mfma:
            groups = N * KV
            if groups >= attn_fill_groups():
                part_size = -(-span // 32) * 32  # enough workgroups without partitions: no merge
            else:
                part_size = min(MFMA_PARTITIONS, key=lambda part: _partition_cost(groups, span, part))
        else:
            groups, part_size = N * KV * max(1, (G + 7) // 8), 256
            while part_size < span and groups * math.ceil(span / part_size) > 2048:
                part_size *= 2
    if mfma and part_size % 32:
        raise KernelError("attention: partitions of the matrix-core kernel are multiples of 32 keys")
    P = max(1, math.ceil(max_context / part_size))
    part_m = part_l = part_acc = None
    if P > 1:
        part_m = torch.empty((N, H, P), dtype=F32, device=device)
        part_l = torch.empty((N, H, P), dtype=F32, device=device)
        part_acc = torch.empty((N, H, P, D), dtype=F32, device=device)
    return part_size, P, part_m, part_l, part_acc


def attn_decode_fresh_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, block_size: int,
                                rotary_dim: int, qk_norm: bool) -> bool:
    """Whether `attn_decode_fresh` takes this case: bfloat16 heads of 64, 128, 192 or 256 with a per-head
    norm, rotated whole, at most 16 query heads to a kv head, pages of a multiple of 16 tokens."""
    return (dtype == BF16 and head_dim % 64 == 0 and head_dim <= 256 and rotary_dim == head_dim and qk_norm
            and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16 and block_size % 16 == 0
            and _decode_mfma_fits(head_dim, num_heads // num_kv_heads))  # fmt: skip


def attn_decode_fresh(qkv, q_weight, k_weight, cos_sin, slots, eps, store_kv, k_pages, v_pages, positions,
                      block_tables, out, num_heads, scale, window, max_context, part_size=None, order=None) -> None:
    """A decode step from the projection's output, in one kernel: what `qk_norm_rope_store` and then
    `attn_single_query` do for tokens that are their own rows (token t reads block table t).

    qkv [T, H + 2 KV, D] bf16; q_weight, k_weight [D] bf16 or fp32; cos_sin [T, D/2, 2] fp32;
    slots [T] int32; store_kv False: queries only, the pages already hold the tokens' keys and values
    (a run that reads another run's cache); out [T, H, D]; order [T] int32: the tokens in the order in
    which the workgroups take them (a permutation; longest contexts first keeps the compute units evenly
    busy when whole contexts are walked), None: as they come."""
    _check(qkv, "qkv", BF16, (None, None, None))
    T, heads, D = qkv.shape
    H = num_heads
    _check(k_pages, "k_pages", BF16, (None, None, None, D))
    _, KV, bs, _ = k_pages.shape
    if heads != H + 2 * KV:
        raise KernelError(f"qkv has {heads} heads, expected {H} + 2 x {KV}")
    _check(v_pages, "v_pages", BF16, (k_pages.shape[0], KV, D, bs))
    _check(out, "out", BF16, (T, H, D))
    _check(positions, "positions", I32, (T,))
    _check(block_tables, "block_tables", I32, (None, None))
    if block_tables.shape[0] < T:
        raise KernelError(f"attention: {T} tokens that are their own rows need as many block tables")
    R = 2 * cos_sin.shape[1] if cos_sin is not None else 0
    if not attn_decode_fresh_supported(BF16, H, KV, D, bs, R, q_weight is not None and k_weight is not None):
        raise KernelError(f"attention from fresh projections: unsupported heads {H}/{KV}, head width {D}, "
                          f"rotary width {R}, page size {bs}, or no per-head norm")  # fmt: skip
    _check(cos_sin, "cos_sin", F32, (T, D // 2, 2))
    _check(q_weight, "q_weight", (F32, BF16), (D,))
    _check(k_weight, "k_weight", q_weight.dtype, (D,))
    w_dtype = q_weight.dtype
    if store_kv:
        _check(slots, "slots", I32, (T,))
    if order is not None:
        _check(order, "order", I32, (T,))
    if T == 0:
        return
    if max_context > block_tables.shape[1] * bs:
        raise KernelError("attention: block tables are shorter than the longest context")
    part_size, P, part_m, part_l, part_acc = _partitions(T, H, KV, D, max_context, window, True, part_size, qkv.device)
    call("as_attn_decode_fresh", _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _DT[w_dtype], _ptr(cos_sin),
         _ptr(slots) if store_kv else 0, float(eps), int(bool(store_kv)), _ptr(k_pages), _ptr(v_pages),
         _ptr(order) if order is not None else 0, T,
         _ptr(positions), _ptr(block_tables), block_tables.shape[1], _ptr(out), _ptr(part_m), _ptr(part_l),
         _ptr(part_acc), H, KV, D, bs, float(scale), int(window), part_size, P, _stream())  # fmt: skip


PREFILL_TILE_QUERIES = 64  # queries of one work item of the prefill kernel
PREFILL_MAX_HEAD_DIM = 256  # four stages of 32 keys and values of such heads fill 128 KB of LDS


def attn_prefill_supported(dtype, head_dim: int, block_size: int) -> bool:
    """Whether `attn_prefill` takes this case; if not, the rows go through `attn_single_query`."""
    return dtype == BF16 and head_dim % 32 == 0 and head_dim <= PREFILL_MAX_HEAD_DIM and block_size % 16 == 0


# The prefill attention has two variants: a wave owns 32 queries of a head (two column tiles of 16), four waves two
# heads' 64 queries; or a wave owns 16 and four waves one head's 64, which makes twice the workgroups with half the
# arithmetic each for the same keys and values brought into LDS.  And a step of few work items lasts as long as its
# longest (a portion of 512 tokens behind 15,872 cached ones is 128 workgroups of 256 rounds of 64 keys on a GPU with
# places for 512): every item may come as several workgroups, the items of more rounds than a piece has cut along
# their keys into such pieces and merged by a second kernel (csrc/attention.hip, PrefillSplit).
#
# Which of the two and how many pieces is chosen by a cost in microseconds, fitted to the kernel's times on 96 steps
# (portions of 64 to 4,096 tokens behind 0 to 15,872 cached ones, lone prompts of 128 to 16,384 tokens; 16, 32, 40 and
# 64 heads of 128 on 8 kv heads; 256 compute units; keys and values of 24 layers in turn, so that they come from
# memory): a round costs a workgroup of the first kind 1.5 us when it has a compute unit to itself and 2.2 us when it
# shares one, of the second kind 1.25 and 1.4 us; workgroups beyond the places wait for one, in whole turns when the
# items are equally long and evenly when they are of every length (a lone prompt: one round up to all); the merge
# costs 6 us and what it writes and reads.  What the cost picks is within 1 per cent of the best of the 12 choices on
# average there and 22 per cent at worst (the rule it replaces, cut only while pieces x items fit the places and 16
# queries to a wave only while the workgroups are fewer than the compute units: 2.6 per cent and 38; 512 tokens
# behind 15,872 of Qwen3-8B sizes 213 -> 173 us, of Qwen3-14B sizes 337 -> 268).
PREFILL_QUERY_TILES = None  # 1 or 2 to force a variant (measurements and tests); None: by the cost
PREFILL_PIECES = None  # a number to force that many pieces (1: none; measurements and tests); None: by the cost
PREFILL_PIECE_CHOICES = (1, 2, 3, 4, 6, 8)
PREFILL_MIN_PIECE_ROUNDS = 8  # a piece has at least this many rounds (at 24 rounds in all the merge costs what the cut gains)


def _prefill_units(query_tiles: int, group: int) -> int:
    """Workgroups of four waves that share a tile's queries of one kv head."""
    return -(-(64 // (16 * query_tiles)) * group // 4)


def _prefill_cost(num_tiles: int, H: int, KV: int, D: int, rounds: int, mean_rounds: float, query_tiles: int,
                  pieces: int, tokens: int) -> float:  # fmt: skip
    """Microseconds, roughly, of a prompt step's attention: `num_tiles` tiles of 64 queries, the longest item of
    `rounds` rounds of 64 keys, the items of `mean_rounds` on average."""
    group, wide = H // KV, D / 128
    alone, shared = ((1.5, 2.2) if query_tiles == 2 else (1.25, 1.4))
    per_cu = 2 if D <= 128 else 1  # the rings of wider heads leave room for one workgroup
    if per_cu == 1:
        shared = alone
    places = per_cu * compute_units()
    workgroups = num_tiles * KV * _prefill_units(query_tiles, group) * pieces
    piece_rounds = -(-rounds // pieces)
    if workgroups <= compute_units():
        cost = piece_rounds * alone
    elif workgroups <= places:
        cost = piece_rounds * shared
    else:
        work = num_tiles * KV * (64 // (16 * query_tiles)) * group / 4 * pieces  # in full workgroups
        spread = min(1.0, max(0.0, 2.0 * (1.0 - mean_rounds / rounds)))  # 0: all items as long as the longest; 1: of every length
        evenly = max(piece_rounds * shared, (work * mean_rounds / pieces / places + 0.5 * piece_rounds) * shared)
        in_turns = -(-workgroups // places) * piece_rounds * shared
        cost = spread * evenly + (1.0 - spread) * in_turns
    cost *= wide
    if pieces > 1:
        cost += 6.0 + tokens * H * pieces * D * 8 / 2e6  # partial results written and read at 2 TB/s
    return cost + 6.0


def _prefill_plan(num_tiles: int, H: int, KV: int, D: int, max_context: int, window: int = 0, query_tiles=None,
                  tile_keys: int = 0) -> tuple:  # fmt: skip
    """(query tiles of a wave, pieces, rounds of a piece) for a prompt step; pieces 1 (and 0 rounds): nothing is cut.
    tile_keys: the keys that the tiles' last queries see, added up (0: not known; the tiles are then taken to be one
    request's last ones).  Every layer of a step asks the same question: the answers are kept."""
    if query_tiles is None:
        query_tiles = PREFILL_QUERY_TILES
    return _prefill_plan_of(num_tiles, H, KV, D, max_context, window, query_tiles, tile_keys, PREFILL_PIECES, compute_units())


@functools.lru_cache(maxsize=1024)
def _prefill_plan_of(num_tiles, H, KV, D, max_context, window, query_tiles, tile_keys, forced_pieces, units) -> tuple:
    span = min(max_context, window + 64) if window > 0 else max_context  # the keys that the longest item walks
    rounds = max(1, -(-span // 64))
    if tile_keys > 0:
        mean_rounds = min(rounds, max(1.0, tile_keys / num_tiles / 64))
    else:
        mean_rounds = max(rounds - num_tiles / 2, rounds / 2)
    kinds = (2, 1) if query_tiles is None else (int(query_tiles),)
    if forced_pieces is not None:
        cuts = (max(1, min(int(forced_pieces), rounds // 2)),)
    else:
        cuts = tuple(c for c in PREFILL_PIECE_CHOICES if c == 1 or rounds // c >= PREFILL_MIN_PIECE_ROUNDS)
    tokens = 64 * num_tiles
    kind, pieces = min(((k, c) for k in kinds for c in cuts),
                       key=lambda kc: _prefill_cost(num_tiles, H, KV, D, rounds, mean_rounds, kc[0], kc[1], tokens))  # fmt: skip
    return (kind, pieces, -(-rounds // pieces)) if pieces > 1 else (kind, 1, 0)


def attn_prefill(q, k_pages, v_pages, tiles, block_tables, out, scale, window, max_context, query_tiles=None,
                 tile_keys: int = 0) -> None:  # fmt: skip
    """Causal attention of prompt portions over the paged cache, bfloat16, on the matrix cores.

    tiles [Nt, 4] int32: (first flat token, count <= 64, block-table row, position of the first
    token) of up to 64 consecutive tokens of one request; the keys of these tokens are already in
    the pages.  max_context: host bound on the last position + 1 of any tile.
    query_tiles: column tiles of 16 queries that a wave owns, 2 or 1; None: chosen here.
    tile_keys: the sum over the tiles of (position of the first token + count), if the caller knows it: how the
    work is cut is chosen better with it (speed only)."""
    _check(q, "q", BF16, (None, None, None))
    T, H, D = q.shape
    _check(out, "out", BF16, (T, H, D))
    _check(k_pages, "k_pages", BF16, (None, None, None, D))
    _, KV, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", BF16, (k_pages.shape[0], KV, D, bs))
    _check(tiles, "tiles", I32, (None, 4))
    _check(block_tables, "block_tables", I32, (None, None))
    if tiles.shape[0] == 0:
        return
    if H % KV or not attn_prefill_supported(q.dtype, D, bs):
        raise KernelError(f"prefill attention: unsupported heads {H}/{KV}, head width {D} or page size {bs}")
    if max_context > block_tables.shape[1] * bs:
        raise KernelError("attention: block tables are shorter than the longest context")
    query_tiles, pieces, piece_rounds = _prefill_plan(tiles.shape[0], H, KV, D, max_context, window, query_tiles, tile_keys)
    cut = part_ml = part_acc = None
    if pieces > 1:
        cut = torch.empty(tiles.shape[0] * KV * _prefill_units(query_tiles, H // KV), dtype=I32, device=q.device)
        part_ml = torch.empty((T, H, pieces, 2), dtype=F32, device=q.device)
        part_acc = torch.empty((T, H, pieces, D), dtype=F32, device=q.device)
    call("as_attn_prefill_mfma", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(tiles), tiles.shape[0],
         _ptr(block_tables), block_tables.shape[1], _ptr(out), H, KV, D, bs, float(scale), int(window),
         int(query_tiles), pieces, piece_rounds, _ptr(cut), _ptr(part_ml), _ptr(part_acc), _stream())  # fmt: skip


SKINNY_MAX_ROWS = 16  # up to here the bf16 product streams the weights through our own kernel
# 17 to 32 rows: the persistent kernel keeps two row tiles in registers up to this K ...
SKINNY_TWO_MAX_ROWS, SKINNY_TWO_MAX_K = 32, 4096
# ... and pays while the activations, which EVERY workgroup reads whole, stay a fraction of the
# weights' bytes: at 32 rows of 4096 over 256 workgroups (67 MB) the library's product is faster,
# with rows of 1024 (17 MB) this one is, by the two kernels it saves beside.
SKINNY_TWO_MAX_ACT_BYTES = 36 << 20


def _workgroups() -> int:
    """Persistent kernels run one workgroup per compute unit."""
    return compute_units()



def _few_rows(rows: int, k: int, n: int, max_k=None, w=None) -> bool:
    """Whether a product of `rows` rows of width `k` with `n` output columns goes through the
    few-rows kernels of this package.  w: the weights, if known: with a copy in wave order, 17 to 32
    rows are left to the tile products (and the library), which are then the faster ones, also for narrow
    rows (Qwen3-0.6B sizes, batch 32: 12,430 -> 12,580 to 12,750 tokens/s), and so are 9 to 16 rows of a
    model that is wide enough (`_tile_preferred`; Qwen3-8B sizes, batch 16: 3,497 -> 3,594, batch 9: 2,045
    -> 2,106; at 8 rows and fewer the few-rows kernels win: 2,129 against 2,019)."""
    if rows <= 0 or k % 8:
        return False
    if w is not None and _tile_preferred(rows, k, n, w):
        return False
    if rows <= SKINNY_MAX_ROWS:
        return max_k is None or k <= max_k
    strips = min(-(-n // 16), _workgroups())
    return (rows <= SKINNY_TWO_MAX_ROWS and k <= SKINNY_TWO_MAX_K
            and strips * rows * k * 2 <= SKINNY_TWO_MAX_ACT_BYTES)  # fmt: skip


def gemm(a, w, out, choices=None) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T.  fp32: own kernel (true fp32).  bf16: own kernel for few
    rows, the library's matrix product otherwise; `out` may be bf16 or (few rows) fp32.
    w: a tensor, or a `Streamed`.  choices: the `ProductChoices` that says which of the library's kernels
    runs (a model's own; None: the one the process shares)."""
    _check(a, "a", (F32, BF16), (None, None))
    M, K = a.shape
    rows = _rows(w)
    _check(rows, "w", a.dtype, (None, K))
    N = rows.shape[0]
    _check(out, "out", None, (M, N))
    if M == 0:
        return
    if a.dtype == F32:
        _check(out, "out", F32)
        call("as_gemm_f32", _ptr(a), _ptr(rows), _ptr(out), M, N, K, _stream())
        return
    if out.dtype not in (BF16, F32):
        raise KernelError(f"gemm: unsupported output dtype {out.dtype}")
    if _few_rows(M, K, N, w=w if out.dtype == BF16 else None):  # fp32 results (the head): no tile product to prefer
        call("as_gemm_bf16_skinny", _ptr(a), _ptr(rows), _wave_ptr(w), _ptr(out), _DT[out.dtype], M, N, K, 0, _stream())
    else:
        (choices or SHARED).gemm(a, w, out, M, N, K)


# ---- the library's product, called directly -------------------------------------------------
#
# hipBLASLt through `csrc/blas.hip` instead of torch.mm: the same kernels for two thirds of the
# time on the host.  For the row counts that a `ProductChoices` is told to tune (decode steps of 17
# and more requests are padded to a few row counts, which the capture of such a step names, and are
# replayed thousands of times) the library's first candidate is often not its fastest on this GPU, so
# the first calls of such a shape try the candidates in turn, each on the weights of the layer that
# happens to call (cold, as every decode step meets them), timed by events in place; when every
# candidate has run LIBRARY_TRIALS_EACH times (the first run of a kernel is slow), or a capture
# begins, the fastest stays.  The same is done for the token budget of a step and for lengths of
# prompts that a warm-up runs, and a product of any other row count above 64 takes the kernel that
# the nearest tuned row count above it settled on: at 128 rows of Qwen3-8B sizes the library's first
# candidates take 168 us a layer, the fastest of the first sixteen 132 us.
LIBRARY_WORKSPACE_BYTES = 64 << 20
LIBRARY_DECODE_ROWS = 64  # row counts up to here are decode steps' (padded to 32, 48 and 64)
LIBRARY_TRIALS_EACH = 4
_workspace = {}  # device index -> the library's scratch memory, one for the process (its calls follow one another)

# Beside the library's candidates a trial may time this package's plain tile product (9 to 128 rows, K in
# chunks of 256, bf16 out, weights with a copy in wave order) with tiles of 2 and of 4 strips: for qkv
# of Qwen3-8B sizes it takes 12.7 / 14.8 / 16.3 us at 32 / 48 / 64 rows against the library's best 14.7 /
# 17.3 / 17.6; for the 4,096 columns of o the library wins at 32 to 64 rows.  Such a candidate's number
# is OWN_CANDIDATE + its strips.
OWN_CANDIDATE = 1000


def _library_workspace(device):
    """The library's scratch memory on `device`; None inside a capture that finds none yet (nothing is
    allocated for good there)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    space = _workspace.get(index)
    if space is None and not torch.cuda.is_current_stream_capturing():
        space = _workspace[index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return space


def _torch_gemm(a, w, out) -> None:
    w = _rows(w)
    if out.dtype == BF16:
        torch.mm(a, w.t(), out=out)
    else:
        out.copy_(torch.mm(a, w.t()))


def _own_candidates(M, N, K, dtype, w) -> list:
    """w: the weights, to see whether they have a copy in wave order; None: taken for granted."""
    if dtype != BF16 or not _tile_rows(M, K, BF16, TILE_SPLIT_MAX_ROWS) or N % 16:
        return []
    if w is not None and not _wave_ptr(w):
        return []
    return [OWN_CANDIDATE + 2, OWN_CANDIDATE + 4]


def _library_call(a, w, out, M, N, K, candidate) -> None:
    if candidate >= OWN_CANDIDATE:
        if not _wave_ptr(w) or out.dtype != BF16:
            raise KernelError("the tile product was chosen for weights with a copy in wave order and bf16 results")
        call("as_gemm_bf16_tile", _ptr(a), _ptr(_rows(w)), _wave_ptr(w), _ptr(out), 0, _DT[BF16], M, N, K, 0, 0,
             candidate - OWN_CANDIDATE, _stream())  # fmt: skip
        return
    call("as_blas_gemm", _ptr(a), _ptr(_rows(w)), _ptr(out), _DT[out.dtype], M, N, K, candidate,
         _ptr(_library_workspace(a.device)), LIBRARY_WORKSPACE_BYTES, _stream())  # fmt: skip


def prepare_library_adoption() -> bool:
    """Pays the library's one-time cost of finding a kernel by its number (a third of a second) now, not
    at the first prompt of a length that was not tuned.  False while no shape has been planned."""
    return bool(entry("as_blas_prepare_adoption")())


class ProductChoices:
    """Which kernel runs for each shape of the matrix products that the few-rows kernels leave over: one
    of the library's candidates or one of this package's tile products, settled by timed trials for the
    row counts it is told to tune, or always the library's first (`fixed`).  A model owns one (its parts
    hand it to `gemm`), so what is chosen on one model's weights, which row counts are tuned and whether
    choices are fixed belong to that model's engine or tool and to no other in the process; calls that
    name none share `SHARED`."""

    def __init__(self, fixed: bool = False):
        self.fixed = bool(fixed)
        self.choice = {}  # (rows, columns, width, output dtype) -> candidate
        self.trials = {}  # the same key -> a trial under way
        self.tuned_rows = {32, 48, 64}

    def fix(self, fixed: bool = True) -> None:
        """fixed: every shape not settled yet takes the library's first candidate (what torch.mm runs)
        instead of timing the candidates, so that bfloat16 results are the same from process to process.
        Choices already made stay (they were made under the setting of their time)."""
        self.fixed = bool(fixed)
        if fixed:
            self.trials.clear()

    def chosen(self) -> dict:
        """(rows, columns, width, output dtype) -> the candidate that runs, for every shape settled so far
        (-1: torch's own call; OWN_CANDIDATE + strips: this package's tile product); enough to reproduce a
        run's products."""
        return dict(self.choice)

    def tune_rows(self, rows: int) -> None:
        """Also try the candidates for products of this many rows: a row count that comes again and
        again, like the token budget of the steps that carry a portion of a prompt."""
        self.tuned_rows.add(int(rows))

    def trials_pending(self) -> bool:
        """Whether some shape is still trying candidates (a warm-up may then run once more)."""
        return bool(self.trials)

    def gemm(self, a, w, out, M, N, K) -> None:
        key = (M, N, K, out.dtype)
        choice = self.choice.get(key)
        if choice is None:
            capturing = torch.cuda.is_current_stream_capturing()
            if _library_workspace(a.device) is None:
                return _torch_gemm(a, w, out)  # inside a capture, before any call outside one: torch's own call this once
            trial = self.trials.get(key)
            if trial is None:
                count = entry("as_blas_plan")(M, N, K, _DT[out.dtype], LIBRARY_WORKSPACE_BYTES)
                if count == 0:
                    choice = self.choice[key] = -1  # the library offers nothing for this shape through this door
                elif self.fixed or (count == 1 and not _own_candidates(M, N, K, out.dtype, w)):
                    choice = self.choice[key] = 0  # the library's first candidate, which is what torch.mm runs
                elif M not in self.tuned_rows:
                    choice = self._choice_of_tuned_rows(M, N, K, out.dtype)  # a prompt of any length: what its bucket settled on
                    if choice is None:
                        choice = 0  # nothing settled yet: the first candidate for now, asked again at the next call
                    else:
                        self.choice[key] = choice
                else:
                    ids = list(range(count)) + _own_candidates(M, N, K, out.dtype, w)
                    trial = self.trials[key] = {"count": len(ids), "ids": ids, "runs": []}
            if trial is not None:
                if not capturing and not _tried_enough(trial):
                    trial["last"] = (a, w, out)
                    _trial_run(trial, a, w, out, M, N, K)
                    return
                choice = self.choice[key] = _fastest_of(self.trials.pop(key))
        if choice < 0:
            return _torch_gemm(a, w, out)
        if choice >= OWN_CANDIDATE and not _wave_ptr(w):
            choice = 0  # chosen on weights that had a copy in wave order; these have none
        _library_call(a, w, out, M, N, K, choice)

    def _choice_of_tuned_rows(self, M, N, K, dtype):
        """For a product of a row count that is not tuned itself: the kernel that the nearest tuned row
        count above it (of more than 64 rows: a prompt's, not a decode step's) settled on for the same
        weights, as a candidate of this shape; None while that one has not settled, or there is none."""
        above = [rows for rows in self.tuned_rows if rows >= M and rows > LIBRARY_DECODE_ROWS]
        if not above:
            return None
        tuned = min(above)
        settled = self.choice.get((tuned, N, K, dtype))
        if settled is None:
            return None
        if settled < 0:
            return 0
        if settled >= OWN_CANDIDATE:  # this package's tile kernel: for this row count too if it takes it, else the library's first
            return settled if settled in _own_candidates(M, N, K, dtype, None) else 0
        index = entry("as_blas_candidate_index")(tuned, N, K, _DT[dtype], LIBRARY_WORKSPACE_BYTES, settled)
        place = entry("as_blas_adopt")(M, N, K, _DT[dtype], LIBRARY_WORKSPACE_BYTES, index)
        return place if place >= 0 else 0

    def settle(self) -> None:
        """Ends every trial that is under way.  Called before a capture begins, so that the captured
        launches are the ones later replays should make.  A shape that a pass meets once (the head)
        has not come round often enough by then: the rest of its runs are made here, on the operands
        of its last call."""
        for key in list(self.trials):
            trial = self.trials.pop(key)
            a, w, out = trial["last"]
            while not _tried_enough(trial):
                _trial_run(trial, a, w, out, *key[:3])
            torch.cuda.current_stream().synchronize()
            self.choice[key] = _fastest_of(trial)


SHARED = ProductChoices()  # for products whose caller names no choices of its own (tools, tests, toy parts)


def _tried_enough(trial) -> bool:
    return len(trial["runs"]) >= LIBRARY_TRIALS_EACH * trial["count"]


def _trial_run(trial, a, w, out, M, N, K) -> None:
    """Computes the product with the candidate whose turn it is, between two events."""
    candidate = trial["ids"][len(trial["runs"]) % trial["count"]]
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    try:
        _library_call(a, w, out, M, N, K, candidate)
    except KernelError:  # a candidate that does not run; the first one does
        trial["runs"].append((candidate, None, None))
        _library_call(a, w, out, M, N, K, 0)
        return
    end.record()
    trial["runs"].append((candidate, start, end))


def _fastest_of(trial) -> int:
    """The candidate whose runs took least on average, among the runs that were timed and have
    finished and leaving out each candidate's first (which loads the kernel); 0 if none."""
    times = {}
    for candidate, start, end in trial["runs"]:
        if start is not None and end.query():
            times.setdefault(candidate, []).append(start.elapsed_time(end))
    best, best_time = 0, float("inf")
    for candidate, took in times.items():
        rest = took[1:] or took
        mean = sum(rest) / len(rest)
        if mean < best_time:
            best, best_time = candidate, mean
    return best


# ---- 17 to 128 rows: tiles of weight rows with the activations staged in LDS --------------------
# (above 64 rows in row tiles of 96 and 128.  At 128 rows the library needs 42 us for Qwen3-8B's down
# projection and 21 for o, the split product 24 on average; the gated product of 96 and 128 rows lost to
# the library's with the activation after it while it read the weights from rows, 51 and 61 us against
# 48 and 56, and wins by a little since it reads them in wave order: batch 96 9,507 -> 9,587 tokens/s)
TILE_MAX_ROWS = 128
TILE_SPLIT_MAX_ROWS = 128
TILE_CHUNK = 256  # K comes in chunks of this many


TILE_MIN_ROWS = 9  # up to 8 rows the few-rows kernels are the faster ones in any case (one row tile of 16, half of it padding)
# ... and at 9 to 16 rows while the model is narrow: with their residual sum and norm folded in they save two
# launches a layer, which a small model's step is made of (decode at batch 16, tile products from 9 rows against
# from 17: Qwen3-0.6B sizes 8,391 against 9,082 tokens/s, -1.7B 7,030 against 7,311, -4B 4,697 against 4,499,
# -8B 3,594 against 3,497, -14B 2,311 against 2,069)
TILE_FROM_9_MIN_WIDTH = 2560


def _tile_rows(rows: int, k: int, dtype, most: int = TILE_MAX_ROWS) -> bool:
    return dtype == BF16 and TILE_MIN_ROWS <= rows <= most and k % TILE_CHUNK == 0


def _tile_preferred(rows: int, k: int, n: int, w) -> bool:
    """Whether a product of 9 to 32 rows that the few-rows kernels could take is left to the tile products
    (and the library with them as candidates): weights with a copy in wave order, a K in whole chunks, and
    above 16 rows or a model wide enough (the narrower of k and n is the stream's width in all four
    products of a layer)."""
    return bool(_wave_ptr(w)) and _tile_rows(rows, k, BF16) and (rows > SKINNY_MAX_ROWS or min(k, n) >= TILE_FROM_9_MIN_WIDTH)


def _gated_tile_strips(rows: int, outputs: int) -> int:
    """Strips of 16 weight rows (gate and up together) per workgroup of the gated tile kernel: a
    workgroup loads 16 rows of weights per strip and `rows` rows of activations, and the workgroups
    run in rounds of one per compute unit; the width with the least to load on the longest path."""
    def cost(strips):
        tiles = -(-outputs // (8 * strips))
        return -(-tiles // compute_units()) * (16 * strips + rows)

    return min((8, 6, 4, 2), key=cost)


def gemm_split_plan(rows: int, n: int, k: int, dtype):
    """(strips, splits) of `gemm_split` for a product of these sizes, or None where it has no kernel:
    tiles of 64 weight rows, and K cut into as many ranges (of whole chunks, as equal as they come) as
    fill the compute units with those tiles."""
    if not _tile_rows(rows, k, dtype, TILE_SPLIT_MAX_ROWS) or n % 4:
        return None
    strips = 4
    tiles = -(-n // (16 * strips))
    chunks = k // TILE_CHUNK
    want = max(1, min(chunks, compute_units() // tiles))
    per = -(-chunks // want)  # chunks of a range; the last range may have fewer (38 chunks in 6 ranges: 7, 7, 7, 7, 7, 3)
    return strips, -(-chunks // per)


def gemm_split(a, w, plan=None):
    """The fp32 partial sums [splits, M, N] of a[M, K] @ w[N, K]^T with K cut into `splits` ranges;
    whoever takes them adds them up (`rmsnorm(..., split_sums=)`).  bf16, 17 to 128 rows."""
    _check(a, "a", BF16, (None, None))
    M, K = a.shape
    rows = _rows(w)
    _check(rows, "w", BF16, (None, K))
    N = rows.shape[0]
    plan = plan or gemm_split_plan(M, N, K, a.dtype)
    if plan is None:
        raise KernelError(f"gemm_split: {M} rows, {K} -> {N} have no kernel")
    strips, splits = plan
    sums = torch.empty((splits, M, N), dtype=F32, device=a.device)
    call("as_gemm_bf16_tile", _ptr(a), _ptr(rows), _wave_ptr(w), 0, _ptr(sums), _DT[F32], M, N, K, 0, splits, strips, _stream())
    return sums


GATED_MAX_K = 6144  # the widest input the fused product-and-activation kernel keeps in registers


def _gated_two_tiles(rows: int, k: int, w) -> bool:
    """17 to 32 rows through the persistent gated kernel with two row tiles also where the plain products of
    such widths are the library's: it saves the activation kernel and the write and read of gate and up.
    Only for weights without a copy in wave order: with one, the gated tile product is faster at these
    widths (Qwen3-8B sizes: batch 32 5,859 -> 5,980 tokens/s, batch 24 4,659 -> 4,755)."""
    return (not _wave_ptr(w) or not _tile_rows(rows, k, BF16)) and SKINNY_MAX_ROWS < rows <= SKINNY_TWO_MAX_ROWS \
        and k <= SKINNY_TWO_MAX_K and k % 8 == 0  # fmt: skip


def gemm_silu_mul(a, w, out, choices=None) -> None:
    """out[M, I] = silu(a @ w[:I]^T) * (a @ w[I:]^T) for w[2 I, K]: the gate and up products and
    the activation.  bf16 with few rows: one kernel, the products rounded to bf16 before the
    activation exactly as the two-kernel path does; otherwise the product, then the activation."""
    _check(a, "a", (F32, BF16), (None, None))
    M, K = a.shape
    _check(out, "out", a.dtype, (M, None))
    inter = out.shape[1]
    rows = _rows(w)
    _check(rows, "w", a.dtype, (2 * inter, K))
    if M == 0:
        return
    if a.dtype == BF16 and (_few_rows(M, K, inter, GATED_MAX_K, w=w) or _gated_two_tiles(M, K, w)):
        call("as_gemm_bf16_gated", _ptr(a), _ptr(rows), _wave_ptr(w), _ptr(out), M, inter, K, _stream())
        return
    if _tile_rows(M, K, a.dtype):
        call("as_gemm_bf16_tile", _ptr(a), _ptr(rows), _wave_ptr(w), _ptr(out), 0, _DT[BF16], M, inter, K, 1, 0,
             _gated_tile_strips(M, inter), _stream())  # fmt: skip
        return
    gate_up = torch.empty((M, 2 * inter), dtype=a.dtype, device=a.device)
    gemm(a, w, gate_up, choices)
    silu_mul(gate_up, out)


def gemm_link_supported(rows: int, n_out: int, k: int, dtype, w=None) -> bool:
    """Whether `gemm_link` and, for its result, `gemm_scaled` exist: bf16, few rows, widths the
    kernels take (n_out is the width of the stream, which is the next product's input).  w: the
    producer's weights, if known (see `_few_rows`)."""
    if dtype != BF16 or rows <= 0 or k % 8 or n_out % 8 or n_out > GATED_MAX_K:
        return False
    if w is not None and _tile_preferred(rows, k, n_out, w):
        return False
    if rows <= SKINNY_MAX_ROWS:
        return True
    # two row tiles: the producer reads its activations once per strip of 16 outputs (whole rows
    # for every workgroup of the persistent kernel, and for every strip beyond its K), the consumer
    # keeps rows of n_out in registers in each of its workgroups
    producer_strips = -(-n_out // 16) if k > SKINNY_TWO_MAX_K else min(-(-n_out // 16), _workgroups())
    return (rows <= SKINNY_TWO_MAX_ROWS and producer_strips * rows * k * 2 <= SKINNY_TWO_MAX_ACT_BYTES
            and _few_rows(rows, n_out, 16 * _workgroups()))  # fmt: skip


def gemm_link(a, w, x, gain, scaled, ssq) -> None:
    """The last product of a part of a pre-norm layer with the residual sum and the first half of
    the next RMSNorm: x[M, N] (fp32) += bf16(a @ w^T); scaled[M, N] = bf16(x * gain), the next
    product's input without its 1/rms factor; ssq[M, ceil(N / 16)] = sums of x^2 per 16 columns.
    a, w bf16; gain fp32 [N]."""
    _check(a, "a", BF16, (None, None))
    M, K = a.shape
    rows = _rows(w)
    _check(rows, "w", BF16, (None, K))
    N = rows.shape[0]
    if not gemm_link_supported(M, N, K, a.dtype):
        raise KernelError(f"gemm_link: {M} rows, {K} -> {N} have no fused kernel")
    _check(x, "x", F32, (M, N))
    _check(gain, "gain", F32, (N,))
    _check(scaled, "scaled", BF16, (M, N))
    _check(ssq, "ssq", F32, (M, -(-N // 16)))
    call("as_gemm_bf16_link", _ptr(a), _ptr(rows), _wave_ptr(w), _ptr(x), _ptr(gain), _ptr(scaled), _ptr(ssq), M, N, K,
         _stream())  # fmt: skip


def gemm_scaled(scaled, ssq, eps, w, out, gated=False) -> None:
    """The first product of the part that follows a `gemm_link`: out = (scaled @ w^T) / rms with
    rms^2 = sum(ssq) / K + eps per row (gated: silu of the first half of w's rows times the
    second half, both scaled and rounded to bf16 first).  scaled [M, K], w, out bf16."""
    _check(scaled, "scaled", BF16, (None, None))
    M, K = scaled.shape
    _check(ssq, "ssq", F32, (M, -(-K // 16)))
    _check(out, "out", BF16, (M, None))
    N = out.shape[1]
    rows = _rows(w)
    _check(rows, "w", BF16, (2 * N if gated else N, K))
    if not gemm_link_supported(M, K, 8, BF16):
        raise KernelError(f"gemm_scaled: {M} rows of width {K} have no fused kernel")
    call("as_gemm_bf16_scaled", _ptr(scaled), _ptr(ssq), ssq.shape[1], float(eps), _ptr(rows), _wave_ptr(w), _ptr(out), M, N, K,
         int(bool(gated)), _stream())  # fmt: skip


SAMPLE_MAX_TOP_K = 1024


def argmax(logits, out) -> None:
    """out[b] = index of the largest logit of row b (the lowest index among equals)."""
    _check(logits, "logits", F32, (None, None))
    _check(out, "out", I32, (logits.shape[0],))
    call("as_argmax", _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1], _stream())


def apply_penalty(logits, rows, cols, amounts) -> None:
    """logits[rows[i], cols[i]] -= amounts[i] for distinct (row, col) pairs."""
    _check(logits, "logits", F32, (None, None))
    n = rows.shape[0]
    _check(rows, "rows", I32, (n,))
    _check(cols, "cols", I32, (n,))
    _check(amounts, "amounts", F32, (n,))
    call("as_apply_penalty", _ptr(logits), _ptr(rows), _ptr(cols), _ptr(amounts), n, logits.shape[1], _stream())


SAMPLE_SPLIT_MAX_TOP_K = 64  # up to here a row's candidates are found by 32 workgroups instead of one


def sample(logits, temperature, top_k, top_p, seeds, counters, out, max_top_k=None) -> None:
    """One token per row: top-k (0: all), temperature (0: greedy), top-p, seeded draw.

    temperature, top_p fp32 [B]; top_k, counters int32 [B]; seeds int64 [B]; out int32 [B].
    A top_k of 0 (or >= vocabulary) keeps all tokens; up to SAMPLE_MAX_TOP_K the candidates are
    ranked (the lower index first among equals); beyond, every token at least as large as the k-th
    largest stays (equal ones together).  max_top_k: the caller's promise that every row keeps between 1
    and this many candidates (a greedy row keeps 1); up to SAMPLE_SPLIT_MAX_TOP_K the rows are
    then searched by many workgroups each, with the same result."""
    _check(logits, "logits", F32, (None, None))
    B = logits.shape[0]
    _check(temperature, "temperature", F32, (B,))
    _check(top_k, "top_k", I32, (B,))
    _check(top_p, "top_p", F32, (B,))
    _check(seeds, "seeds", torch.int64, (B,))
    _check(counters, "counters", I32, (B,))
    _check(out, "out", I32, (B,))
    if max_top_k is not None and 1 <= max_top_k <= SAMPLE_SPLIT_MAX_TOP_K:
        cand = torch.empty((B, 32, SAMPLE_SPLIT_MAX_TOP_K), dtype=torch.int64, device=logits.device)
        counts = torch.empty((B, 32), dtype=I32, device=logits.device)
        call("as_sample_split", _ptr(logits), B, logits.shape[1], _ptr(temperature), _ptr(top_k), _ptr(top_p),
             _ptr(seeds), _ptr(counters), _ptr(cand), _ptr(counts), _ptr(out), _stream())  # fmt: skip
        return
    call("as_sample", _ptr(logits), B, logits.shape[1], _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
         _ptr(counters), _ptr(out), _stream())  # fmt: skip


def topk(logits, k, values, indices) -> None:
    """Sorted k largest of each row: values fp32 [B, k], indices int32 [B, k]."""
    _check(logits, "logits", F32, (None, None))
    B, V = logits.shape
    if not 0 < k <= min(V, SAMPLE_MAX_TOP_K):
        raise KernelError(f"top-k of {k} is outside 1..{min(V, SAMPLE_MAX_TOP_K)}")
    _check(values, "values", F32, (B, k))
    _check(indices, "indices", I32, (B, k))
    call("as_topk", _ptr(logits), B, V, k, _ptr(values), _ptr(indices), _stream())


# ---- layers whose parts read one stream side by side -------------------------------------------------


def rmsnorm_multi(x, weight1, weight2, eps, out1, out2=None, delta1=None, delta2=None, rows=None, update_x=True) -> None:
    """v = x[s] + (delta1[s] + delta2[s]) (either may be absent), s = rows[r] or r; out1[r] = norm(v) * weight1 and,
    if given, out2[r] = norm(v) * weight2, the root mean square taken once; x fp32 [T, n] receives v when
    `update_x` and something was added."""
    _check(x, "x", F32, (None, None))
    T, n = x.shape
    n_out = T
    if rows is not None:
        _check(rows, "rows", I32, (None,))
        n_out = rows.shape[0]
    _check(out1, "out1", (F32, BF16), (n_out, n))
    _check(weight1, "weight1", (F32, BF16), (n,))
    if out1.dtype == F32 and weight1.dtype != F32:
        raise KernelError("fp32 norm needs an fp32 weight")
    if (out2 is None) != (weight2 is None):
        raise KernelError("a second output and a second weight come together")
    if out2 is not None:
        _check(out2, "out2", out1.dtype, (n_out, n))
        _check(weight2, "weight2", weight1.dtype, (n,))
    for name, d in (("delta1", delta1), ("delta2", delta2)):
        if d is not None:
            _check(d, name, out1.dtype, (T, n))
    call("as_rmsnorm_multi", _ptr(x), _ptr(delta1), _ptr(delta2), _ptr(rows), _ptr(weight1), _ptr(weight2),
         _DT[weight1.dtype], float(eps), _ptr(out1), _ptr(out2), _DT[out1.dtype], n_out, n, int(bool(update_x)), _stream())  # fmt: skip


def head_norm_store(proj, q_off, k_off, v_off, num_heads, num_kv_heads, dim, vdim, q_weight, k_weight, eps, slots,
                    q_out, k_pages, v_pages, store_kv=True, cos_sin=None) -> None:  # fmt: skip
    """Heads cut out of a wider projection's output proj [T, ld] (queries at column q_off, keys at k_off, both
    `dim` wide; values at v_off, `vdim` wide): per-head RMS norm of queries and keys (weights [dim], or none), their
    rotation where `cos_sin` (fp32 [T, R/2, 2]) is given (the pairs (i, i + R/2) of a head's first R coordinates;
    values are never turned, so v_off = k_off stores the unturned keys as values), and the cache store.  Every head is laid out Dp = q_out.shape[2] >= max(dim, vdim) wide, zero where
    it has no coordinate: q_out [T, H, Dp], k_pages [pages, KV, bs, Dp], v_pages [pages, KV, Dp, bs]."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H, KV = num_heads, num_kv_heads
    _check(q_out, "q_out", proj.dtype, (T, H, None))
    Dp = q_out.shape[2]
    if Dp < max(dim, vdim) or min(q_off, k_off, v_off) < 0 or q_off + H * dim > ld or k_off + KV * dim > ld \
            or v_off + KV * vdim > ld:  # fmt: skip
        raise KernelError("head_norm_store: heads lie outside the projection's columns or the padded head width")
    w_dtype = proj.dtype
    if q_weight is not None:
        _check(q_weight, "q_weight", (F32, BF16), (dim,))
        _check(k_weight, "k_weight", q_weight.dtype, (dim,))
        w_dtype = q_weight.dtype
        if proj.dtype == F32 and w_dtype != F32:
            raise KernelError("fp32 q/k norm needs fp32 weights")
    elif k_weight is not None:
        raise KernelError("q and k norm weights come together")
    bs = 1
    if store_kv:
        _check(slots, "slots", I32, (T,))
        _check(k_pages, "k_pages", proj.dtype, (None, KV, None, Dp))
        bs = k_pages.shape[2]
        _check(v_pages, "v_pages", proj.dtype, (k_pages.shape[0], KV, Dp, bs))
    R = 0
    if cos_sin is not None:
        _check(cos_sin, "cos_sin", F32, (T, None, 2))
        R = 2 * cos_sin.shape[1]
        if R > dim or R < 2:
            raise KernelError(f"head_norm_store: {R} turned coordinates in a head of {dim}")
    call("as_head_norm_store", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, H, KV, dim, vdim, Dp,
         _ptr(q_weight), _ptr(k_weight), _DT[w_dtype], float(eps), _ptr(slots) if store_kv else 0, _ptr(q_out),
         _ptr(k_pages) if store_kv else 0, _ptr(v_pages) if store_kv else 0, bs, int(bool(store_kv)), T,
         _ptr(cos_sin), R, _stream())  # fmt: skip


def whole_norm_store(proj, q_off, k_off, v_off, num_heads, num_kv_heads, dim, vdim, slots, q_out, k_pages, v_pages,
                     store_kv=True, biases=None, gains=None, eps: float = 0.0, cos_sin=None, v_keep=None,
                     v_mode: str = "none", lam: float = 0.0) -> None:  # fmt: skip
    """`head_norm_store` for heads that are normed over their whole projection.  biases: (q [H dim], k [KV dim], v [KV
    vdim]) fp32, added to the projection's output first, or None.  gains: (q [H dim], k [KV dim]) fp32: queries and keys
    are divided by the root mean square over ALL their heads (eps inside the root) and multiplied by the gains; None: no
    norm.  cos_sin: the rotation (after the norm), as in `head_norm_store`.  v_mode "keep": the values (bias added) are
    also written to v_keep fp32 [T, KV vdim]; "mix": (1 - lam) v + lam v_keep[t] is stored instead of v."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H, KV = num_heads, num_kv_heads
    _check(q_out, "q_out", proj.dtype, (T, H, None))
    Dp = q_out.shape[2]
    if Dp < max(dim, vdim) or min(q_off, k_off, v_off) < 0 or q_off + H * dim > ld or k_off + KV * dim > ld \
            or v_off + KV * vdim > ld:  # fmt: skip
        raise KernelError("whole_norm_store: heads lie outside the projection's columns or the padded head width")
    qb = kb = vb = qw = kw = None
    if biases is not None:
        qb, kb, vb = biases
        for name, t, n in (("q bias", qb, H * dim), ("k bias", kb, KV * dim), ("v bias", vb, KV * vdim)):
            _check(t, name, F32, (n,))
    if gains is not None:
        qw, kw = gains
        _check(qw, "q gain", F32, (H * dim,))
        _check(kw, "k gain", F32, (KV * dim,))
    bs = 1
    if store_kv:
        _check(slots, "slots", I32, (T,))
        _check(k_pages, "k_pages", proj.dtype, (None, KV, None, Dp))
        bs = k_pages.shape[2]
        _check(v_pages, "v_pages", proj.dtype, (k_pages.shape[0], KV, Dp, bs))
    R = 0
    if cos_sin is not None:
        _check(cos_sin, "cos_sin", F32, (T, None, 2))
        R = 2 * cos_sin.shape[1]
        if R > dim or R < 2:
            raise KernelError(f"whole_norm_store: {R} turned coordinates in a head of {dim}")
    modes = {"none": 0, "keep": 1, "mix": 2}
    if v_mode not in modes:
        raise KernelError(f"whole_norm_store: values are handled as one of {sorted(modes)}, not {v_mode!r}")
    if modes[v_mode]:
        _check(v_keep, "v_keep", F32, (T, KV * vdim))
    call("as_whole_norm_store", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, H, KV, dim, vdim, Dp, _ptr(qb),
         _ptr(kb), _ptr(vb), _ptr(qw), _ptr(kw), float(eps), _ptr(cos_sin), R, _ptr(v_keep) if modes[v_mode] else 0,
         modes[v_mode], float(lam), _ptr(slots) if store_kv else 0, _ptr(q_out), _ptr(k_pages) if store_kv else 0,
         _ptr(v_pages) if store_kv else 0, bs, int(bool(store_kv)), T, _stream())  # fmt: skip


STREAMS_MAX = 16


def streams_step(xs, first=None, y=None, mix=None, out_c=None, mult: float = 1.0, in_c=None, gain=None, eps: float = 0.0,
                 normed=None, total=None) -> None:  # fmt: skip
    """One step between two parts of a model with several residual streams xs fp32 [T, S, n] (updated in place).
    first [T, n] fp32: the streams do not exist yet, all of them are `first`.  y [T, n] (compute dtype): the pending
    write xs[:, r] <- sum_s mix[s, r] xs[:, s] + mult out_c[r] y (mix fp32 [S, S], None: the identity; out_c fp32 [S]).
    in_c fp32 [S] with gain fp32 [n] and normed [T, n] (compute dtype): normed = rmsnorm(sum_s in_c[s] xs[:, s]) * gain.
    total fp32 [T, n]: receives sum_s xs[:, s]."""
    _check(xs, "xs", F32, (None, None, None))
    T, S, n = xs.shape
    if not 1 <= S <= STREAMS_MAX:
        raise KernelError(f"1 to {STREAMS_MAX} streams, not {S}")
    dtype = None
    if first is not None:
        _check(first, "first", F32, (T, n))
    if y is not None:
        _check(y, "y", (F32, BF16), (T, n))
        dtype = y.dtype
        _check(out_c, "out_c", F32, (S,))
        if mix is not None:
            _check(mix, "mix", F32, (S, S))
    if (in_c is None) != (normed is None):
        raise KernelError("streams_step: the read's weights and the normed rows come together")
    if normed is not None:
        _check(normed, "normed", (F32, BF16) if dtype is None else dtype, (T, n))
        dtype = normed.dtype
        _check(in_c, "in_c", F32, (S,))
        _check(gain, "gain", F32, (n,))
    if total is not None:
        _check(total, "total", F32, (T, n))
    call("as_streams_step", _ptr(xs), _ptr(first), S, n, _ptr(y), _DT[dtype if dtype is not None else F32], _ptr(mix),
         _ptr(out_c), float(mult), _ptr(in_c), _ptr(gain), float(eps), _ptr(normed), _ptr(total), T, _stream())  # fmt: skip


def gated_add_norm(x, y, gate, gate_off, bias, mult, weight, eps, out, rows=None, update_x=True, other=None,
                   join=None) -> None:  # fmt: skip
    """The fp32 stream x [T, n] takes a part's gated, scaled output and is normed, in one kernel:
    x[s] += mult * sigmoid(gate[s, gate_off:gate_off + n] + bias) * y[s]   (y None: nothing is added)
    out[r] = x[s] / sqrt(mean(x[s]^2) + eps) * weight                      (weight None: no norm; out fp32 or y's dtype)
    join[r] = [x[s] | other[s]] in the compute dtype                        (join None: none)
    with s = rows[r] (or r).  y [T, n] and gate [T, ld] are a part's output and the logits of its gate."""
    _check(x, "x", F32, (None, None))
    T, n = x.shape
    n_out = T
    if rows is not None:
        _check(rows, "rows", I32, (None,))
        n_out = rows.shape[0]
    dtype = None
    ld = 0
    if y is not None:
        _check(y, "y", (F32, BF16), (T, n))
        dtype = y.dtype
        _check(gate, "gate", dtype, (T, None))
        ld = gate.shape[1]
        if gate_off < 0 or gate_off + n > ld:
            raise KernelError("gated_add_norm: the gate lies outside its product's columns")
    if join is not None:
        _check(join, "join", (F32, BF16) if dtype is None else dtype, (n_out, 2 * n))
        _check(other, "other", F32, (T, n))
        dtype = join.dtype
    w_dtype = None
    for name, v in (("weight", weight), ("bias", bias)):
        if v is not None:
            _check(v, name, (F32, BF16) if w_dtype is None else w_dtype, (n,))
            w_dtype = v.dtype
    if weight is not None:
        _check(out, "out", (F32, BF16), (n_out, n))
        if dtype is None:
            dtype = out.dtype if out.dtype == BF16 else weight.dtype
    if dtype is None:
        return  # nothing to add, to norm or to join
    if w_dtype is None:
        w_dtype = dtype
    if dtype == F32 and w_dtype != F32:
        raise KernelError("gated_add_norm: 32-bit rows need 32-bit gains and biases")
    out_dtype = out.dtype if weight is not None else dtype
    call("as_gated_add_norm", _ptr(x), _ptr(y), _ptr(gate), _DT[dtype], ld, gate_off, _ptr(bias), float(mult),
         _ptr(rows), _ptr(weight), _DT[w_dtype], float(eps), _ptr(out) if weight is not None else 0, _DT[out_dtype],
         n_out, n, int(bool(update_x)), _ptr(other), _ptr(join), _stream())  # fmt: skip


def relu2(a, off, out) -> None:
    """out[t, i] = max(a[t, off + i], 0)^2 for the out.shape[1] columns of a [T, ld] from `off` on."""
    _check(a, "a", (F32, BF16), (None, None))
    T, ld = a.shape
    _check(out, "out", a.dtype, (T, None))
    n = out.shape[1]
    if off < 0 or off + n > ld:
        raise KernelError("relu2: columns outside the input")
    call("as_relu2", _ptr(a), _DT[a.dtype], ld, off, _ptr(out), n, T, _stream())


# ---- attention with mixed heads ----------------------------------------------------------------------

HEADMIX_KEYS = 64  # key slots of a chunk
HEADMIX_MAX_LDS = 96 << 10


def attn_headmix_tile(num_heads: int, head_dim: int, dtype) -> int:
    """The most consecutive queries of a row that one workgroup of `attn_headmix` takes (16, 8, 4, 2 or 1):
    bounded by the accumulators a thread keeps and by LDS; 0: the kernel does not take so many heads."""
    elt = 4 if dtype == F32 else 2
    for tile, most in ((16, 4), (8, 8), (4, 16), (2, 32), (1, 32)):
        if -(-num_heads * head_dim // 256) > most:
            continue
        floats = 2 * num_heads * tile * HEADMIX_KEYS + num_heads * num_heads + 3 * tile * num_heads + HEADMIX_KEYS
        if floats * 4 + 16 + tile * num_heads * head_dim * elt > HEADMIX_MAX_LDS:
            continue
        return tile
    return 0


HEADMIX_MFMA_MAX_LDS = 128 << 10
HEADMIX_MFMA_TILES = 16  # output tiles (kv head, 64 coordinates) that a wave of the matrix-core kernel keeps
HEADMIX_FILL = 2  # workgroups per compute unit up to which an item's keys are cut over several workgroups
HEADMIX_MAX_SPLITS = 64


def _headmix_mfma_lds(H: int, D: int, tq: int) -> int:
    h8 = -(-H // 8) * 8
    scores = -(-H * tq * (HEADMIX_KEYS + 1) // 4) * 4  # rows a little longer than their 64 slots, against bank conflicts
    return (scores + H * h8 + 3 * tq * H + HEADMIX_KEYS) * 4 + 16 + (H * tq * (HEADMIX_KEYS + 8) + tq * H * (D + 8)) * 2


def attn_headmix_mfma_takes(dtype, H: int, KV: int, D: int, block_size: int, tile: int) -> bool:
    """Whether the matrix-core form of `attn_headmix` takes these sizes with items of up to `tile` queries: bf16,
    heads of 32, 64, 96, 128, 192 or 256 coordinates, `tile` queries times the heads of a kv head within a tile's 16 rows,
    pages of 8, 16, 32 or 64 tokens."""
    if dtype != BF16 or H < 1 or KV < 1 or H % KV or H > 64 or tile < 1 or (H // KV) * tile > 16:
        return False
    if (H // KV) & (H // KV - 1):  # 1, 2, 4, 8 or 16 query heads to a kv head: the rows of a tile are cut by shifts
        return False
    if D not in (32, 64, 96, 128, 192, 256) or KV * -(-D // 64) > HEADMIX_MFMA_TILES:
        return False
    if block_size % 8 or block_size > HEADMIX_KEYS or HEADMIX_KEYS % block_size:
        return False
    return _headmix_mfma_lds(H, D, tile) <= HEADMIX_MFMA_MAX_LDS


def attn_headmix_rows(num_heads: int, num_kv_heads: int, head_dim: int, dtype) -> int:
    """How many consecutive queries of a row make a work item of `attn_headmix` for a model of these sizes: what the
    matrix-core kernel packs into a tile's 16 rows beside the heads of a kv head, where it takes the sizes at all
    (whatever the pages: the general kernel serves the pages it does not, taking such an item in turns); else what
    the general kernel takes at once."""
    if attn_headmix_mfma_takes(dtype, num_heads, num_kv_heads, head_dim, 16, 1):
        tile = 16
        while tile > 1 and not attn_headmix_mfma_takes(dtype, num_heads, num_kv_heads, head_dim, 16, tile):
            tile //= 2
        return tile
    return attn_headmix_tile(num_heads, head_dim, dtype)


def _headmix_splits(num_items: int, tile: int, window: int, keep_first: int, max_context: int) -> int:
    """Into how many workgroups an item's keys are cut: one where the items alone fill the GPU, else as many as fill
    it, each with at least one chunk of 64 keys."""
    if max_context <= 0:
        return 1
    keys = max_context if window <= 0 else min(max_context, window + tile - 1 + keep_first + HEADMIX_KEYS)
    chunks = -(-keys // HEADMIX_KEYS) + 1
    want = -(-HEADMIX_FILL * compute_units() // max(1, num_items))
    return max(1, min(chunks, want, HEADMIX_MAX_SPLITS))


def attn_headmix(q, k_pages, v_pages, items, tile: int, positions, tok_row, block_tables, mix, out, scale: float,
                 window: int = 0, keep_first: int = 0, max_context: int = 0, splits: int = None) -> None:  # fmt: skip
    """Softmax attention whose heads' scores are mixed before the softmax: s_h = sum_g mix[h, g] * scale * q_g . k
    (mix fp32 [H, H]; None: no mixing), a query at position i seeing the keys j <= i with i - j < window (0: all)
    or j < keep_first.  q [T, H, D]; out [T, H, Dout], Dout <= D (heads padded to D with zeros lose the padding);
    pages as the other attention kernels read them.
    tile == 1: items [N] int32 are single tokens (positions [T]; tok_row [T] or None where token t is row t);
    else items [N, 4] = (first token, count <= tile, row, first position).
    bf16 with sizes that `attn_headmix_mfma_takes` runs on the matrix cores; max_context (a bound on the positions,
    0: unknown) lets few items' keys be cut over several workgroups (`splits`: forced, for tests)."""
    _check(q, "q", (F32, BF16), (None, None, None))
    T, H, D = q.shape
    _check(out, "out", q.dtype, (T, H, None))
    Dout = out.shape[2]
    if not 1 <= Dout <= D:
        raise KernelError(f"attn_headmix: outputs of {Dout} coordinates from heads of {D}")
    _check(k_pages, "k_pages", q.dtype, (None, None, None, D))
    NB, KV, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q.dtype, (NB, KV, D, bs))
    _check(block_tables, "block_tables", I32, (None, None))
    if H % KV or bs > HEADMIX_KEYS:
        raise KernelError(f"attn_headmix: {H} heads over {KV} kv heads, pages of {bs} (at most {HEADMIX_KEYS})")
    if D % (4 if q.dtype == F32 else 8):
        raise KernelError(f"attn_headmix: heads of {D} are not read 16 bytes at a time")
    if tile not in (1, 2, 4, 8, 16):
        raise KernelError(f"attn_headmix: a tile of {tile} queries (1, 2, 4, 8 or 16)")
    mfma = attn_headmix_mfma_takes(q.dtype, H, KV, D, bs, tile)
    if not mfma and attn_headmix_tile(H, D, q.dtype) < 1:  # (an item of more queries than fit at once is taken in turns)
        raise KernelError(f"attn_headmix: {H} heads of {D} are more than a workgroup keeps at once")
    if tile == 1:
        _check(items, "items", I32, (None,))
        _check(positions, "positions", I32, (T,))
        if tok_row is not None:
            _check(tok_row, "tok_row", I32, (T,))
    else:
        _check(items, "items", I32, (None, 4))
    if mix is not None:
        _check(mix, "mix", F32, (H, H))
    if window < 0 or keep_first < 0:
        raise KernelError("attn_headmix: a window and a number of kept tokens are not negative")
    if mfma:
        N = items.shape[0]
        if splits is None:
            splits = _headmix_splits(N, tile, window, keep_first, max_context)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((N, splits, tile, H, D), dtype=F32, device=q.device)
            part_ml = torch.empty((N, splits, tile, H, 2), dtype=F32, device=q.device)
        call("as_attn_headmix_mfma", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(items), N, tile, int(tile == 1),
             _ptr(positions), _ptr(tok_row), _ptr(block_tables), block_tables.shape[1], _ptr(mix), _ptr(out), H, KV, D,
             Dout, bs, float(scale), int(window), int(keep_first), int(splits), _ptr(part_o), _ptr(part_ml), _stream())  # fmt: skip
        return
    call("as_attn_headmix", _ptr(q), _ptr(k_pages), _ptr(v_pages), _DT[q.dtype], _ptr(items), items.shape[0], tile,
         _ptr(positions), _ptr(tok_row), _ptr(block_tables), block_tables.shape[1], _ptr(mix), _ptr(out), H, KV, D,
         Dout, bs, float(scale), int(window), int(keep_first), _stream())  # fmt: skip


def sigmoid_gate_heads(heads, vdim, gate, gate_off, scale, out, out_off) -> None:
    """out[t, out_off + h * vdim + j] = scale * sigmoid(gate[t, gate_off + h * vdim + j]) * heads[t, h, j], j < vdim;
    gate None: scale * heads, laid side by side."""
    _check(heads, "heads", (F32, BF16), (None, None, None))
    T, H, Dp = heads.shape
    _check(out, "out", heads.dtype, (T, None))
    ld_gate = 0
    if gate is not None:
        _check(gate, "gate", heads.dtype, (T, None))
        ld_gate = gate.shape[1]
        if gate_off < 0 or gate_off + H * vdim > ld_gate:
            raise KernelError("sigmoid_gate_heads: columns outside the gate")
    if vdim > Dp or out_off < 0 or out_off + H * vdim > out.shape[1]:
        raise KernelError("sigmoid_gate_heads: columns outside the output")
    call("as_sigmoid_gate_heads", _ptr(heads), _DT[heads.dtype], H, vdim, Dp, _ptr(gate), ld_gate, gate_off,
         float(scale), _ptr(out), out.shape[1], out_off, T, _stream())  # fmt: skip


# ---- mixers with a fixed-size state --------------------------------------------------------------------


def _check_rows(step_rows, num_tokens):
    tok_row, row_first, row_len, row_start, row_slots = step_rows
    _check(row_first, "row_first", I32, (None,))
    R = row_first.shape[0]
    for name, t in (("row_len", row_len), ("row_start", row_start), ("row_slots", row_slots)):
        _check(t, name, I32, (R,))
    if tok_row is not None:
        _check(tok_row, "tok_row", I32, (num_tokens,))
    elif R < num_tokens:
        raise KernelError("tokens that are their own rows need as many rows")
    return R


def _vector_dtype(proj_dtype, *vectors):
    dtypes = {v.dtype for v in vectors if v is not None}
    if len(dtypes) > 1:
        raise KernelError(f"the small tensors of one part come in one dtype, not {sorted(map(str, dtypes))}")
    dtype = dtypes.pop() if dtypes else proj_dtype
    if dtype not in _DT or (proj_dtype == F32 and dtype != F32):
        raise KernelError(f"small tensors in {dtype} do not go with a projection in {proj_dtype}")
    return dtype


CONV_MAX_TAPS = 8


def short_conv(proj, col0, weight, history, step_rows, out, in_bias=None, bias=None, silu=False, writes=True) -> None:
    """Causal convolution per channel over each row's tokens: out[t, c] = act(sum_i weight[c, i] * in[t - (taps-1-i), c]
    + bias[c]) with in = proj[:, col0 + c] + in_bias[c], zeros before a sequence, and before a row the last taps - 1
    inputs of its request from history [slots, taps - 1, C] (fp32), which then moves on by the row (`writes`).
    step_rows: (tok_row or None, row_first, row_len, row_start, row_slots).  out fp32 [T, C]."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    _check(weight, "weight", (F32, BF16), (None, None))
    C, taps = weight.shape
    if not 1 <= taps <= CONV_MAX_TAPS or col0 < 0 or col0 + C > ld:
        raise KernelError(f"short_conv: {taps} taps (1 to {CONV_MAX_TAPS}) or columns {col0}:{col0 + C} of {ld}")
    w_dtype = _vector_dtype(proj.dtype, weight, in_bias, bias)
    for name, b in (("in_bias", in_bias), ("bias", bias)):
        if b is not None:
            _check(b, name, w_dtype, (C,))
    _check(out, "out", F32, (T, C))
    R = _check_rows(step_rows, T)
    _check(history, "history", F32, (None, max(taps - 1, 0), C) if taps > 1 else None)
    tok_row, row_first, row_len, row_start, row_slots = step_rows
    call("as_short_conv", _ptr(proj), _DT[proj.dtype], ld, col0, C, _ptr(in_bias), _ptr(weight), _ptr(bias),
         _DT[w_dtype], taps, int(bool(silu)), _ptr(history), _ptr(tok_row), _ptr(row_first), _ptr(row_len),
         _ptr(row_start), _ptr(row_slots), _ptr(out), T, R, int(bool(writes)), _stream())  # fmt: skip


def delta_prepare(qkv, num_kv_heads, dim, num_heads, proj, b_off, a_off, a_log, dt_bias, beta, decay) -> None:
    """In place on qkv fp32 [T, C] (G query heads, then G key heads, `dim` wide each, then the values): queries and
    keys become unit vectors (x / sqrt(sum x^2 + 1e-6)), the queries also times dim^(-1/2).  beta [T, H] =
    sigmoid(proj[:, b_off + h]); decay [T, H] = exp(-exp(a_log[h]) * softplus(proj[:, a_off + h] + dt_bias[h]))."""
    _check(qkv, "qkv", F32, (None, None))
    T, C = qkv.shape
    G, H = num_kv_heads, num_heads
    _check(proj, "proj", (F32, BF16), (T, None))
    ld = proj.shape[1]
    if C < 2 * G * dim or min(b_off, a_off) < 0 or max(b_off, a_off) + H > ld:
        raise KernelError("delta_prepare: heads outside the convolution's channels or the projection's columns")
    w_dtype = _vector_dtype(proj.dtype, a_log, dt_bias)
    _check(a_log, "a_log", w_dtype, (H,))
    _check(dt_bias, "dt_bias", w_dtype, (H,))
    _check(beta, "beta", F32, (T, H))
    _check(decay, "decay", F32, (T, H))
    call("as_delta_prepare", _ptr(qkv), C, G, dim, H, _ptr(proj), _DT[proj.dtype], ld, b_off, a_off, _ptr(a_log),
         _ptr(dt_bias), _DT[w_dtype], _ptr(beta), _ptr(decay), T, _stream())  # fmt: skip


def delta_scan(qkv, num_kv_heads, dim, num_heads, vdim, beta, decay, state, step_rows, out, writes=True, slices=0) -> None:
    """The gated delta rule over each row's tokens, per head h (keys and queries of head h // (H / G)):
    S <- decay S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q.  state fp32 [slots, H, dim, vdim]; a row
    that starts at position 0 starts from zero.  qkv as `delta_prepare` left it; out fp32 [T, H, vdim].
    slices: into how many lanes a column of the state is cut (1, 2, 4, 8, 16); 0: chosen so that the step's rows,
    heads and column groups fill the GPU (the results differ by the order of the sums only)."""
    _check(qkv, "qkv", F32, (None, None))
    T, C = qkv.shape
    G, H = num_kv_heads, num_heads
    if H % G or C != 2 * G * dim + H * vdim:
        raise KernelError(f"delta_scan: {C} channels are not 2 x {G} x {dim} + {H} x {vdim}")
    _check(beta, "beta", F32, (T, H))
    _check(decay, "decay", F32, (T, H))
    _check(state, "state", F32, (None, H, dim, vdim))
    _check(out, "out", F32, (T, H, vdim))
    R = _check_rows((None, *step_rows[1:]), 0)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_delta_scan", _ptr(qkv), C, G, dim, H, vdim, _ptr(beta), _ptr(decay), _ptr(state), _ptr(row_first),
         _ptr(row_len), _ptr(row_start), _ptr(row_slots), int(bool(writes)), _ptr(out), R, int(slices), _stream())  # fmt: skip


def delta_finish(o, weight, eps, proj, g_off, act, gate="silu", scale: float = 1.0, out_off: int = 0) -> None:
    """act[t, out_off + h * vdim + j] = scale * o[t, h, j] / rms(o[t, h]) * weight * gate(proj[t, g_off + h * vdim + j]);
    weight [vdim] (shared by the heads) or [H, vdim]; gate "silu" or "sigmoid"; act [T, >= out_off + H * vdim]."""
    _check(o, "o", F32, (None, None, None))
    T, H, vdim = o.shape
    _check(proj, "proj", (F32, BF16), (T, None))
    if g_off < 0 or g_off + H * vdim > proj.shape[1]:
        raise KernelError("delta_finish: the gate lies outside the projection's columns")
    if gate not in ("silu", "sigmoid"):
        raise KernelError(f"delta_finish: a gate is 'silu' or 'sigmoid', not {gate!r}")
    w_dtype = _vector_dtype(proj.dtype, weight)
    per_head = weight.dim() == 2
    _check(weight, "weight", w_dtype, (H, vdim) if per_head else (vdim,))
    _check(act, "act", proj.dtype, (T, None))
    if out_off < 0 or out_off + H * vdim > act.shape[1]:
        raise KernelError("delta_finish: the heads lie outside the output's columns")
    call("as_delta_finish", _ptr(o), H, vdim, _ptr(weight), _DT[w_dtype], int(per_head), float(eps), _ptr(proj),
         _DT[proj.dtype], proj.shape[1], g_off, int(gate == "sigmoid"), float(scale), _ptr(act), act.shape[1], out_off,
         T, _stream())  # fmt: skip


def delta_prepare_channels(qkv, num_kv_heads, dim, num_heads, proj, b_off, steps, a_off, a_log, dt_bias, beta, chan) -> None:
    """As `delta_prepare` for a rule with a decay per head and key channel: chan [T, H, dim] =
    exp(-exp(a_log[h]) * softplus(steps[:, a_off + h * dim + d] + dt_bias[h * dim + d])); a_log [H], dt_bias [H * dim] fp32."""
    _check(qkv, "qkv", F32, (None, None))
    T, C = qkv.shape
    G, H = num_kv_heads, num_heads
    _check(proj, "proj", (F32, BF16), (T, None))
    _check(steps, "steps", proj.dtype, (T, None))
    if C < 2 * G * dim or b_off < 0 or b_off + H > proj.shape[1] or a_off < 0 or a_off + H * dim > steps.shape[1]:
        raise KernelError("delta_prepare_channels: heads outside the convolution's channels or the projections' columns")
    _check(a_log, "a_log", F32, (H,))
    _check(dt_bias, "dt_bias", F32, (H * dim,))
    _check(beta, "beta", F32, (T, H))
    _check(chan, "chan", F32, (T, H, dim))
    call("as_delta_prepare_channels", _ptr(qkv), C, G, dim, H, _ptr(proj), _DT[proj.dtype], proj.shape[1], b_off,
         _ptr(steps), steps.shape[1], a_off, _ptr(a_log), _ptr(dt_bias), _ptr(beta), _ptr(chan), T, _stream())  # fmt: skip


def delta_scan_channels(qkv, num_kv_heads, dim, num_heads, vdim, beta, chan, state, step_rows, out, writes=True, slices=0) -> None:
    """`delta_scan` with a decay per head and key channel, chan fp32 [T, H, dim], acting on the rows of S:
    S <- diag(chan) S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q."""
    _check(qkv, "qkv", F32, (None, None))
    T, C = qkv.shape
    G, H = num_kv_heads, num_heads
    if H % G or C != 2 * G * dim + H * vdim:
        raise KernelError(f"delta_scan_channels: {C} channels are not 2 x {G} x {dim} + {H} x {vdim}")
    _check(beta, "beta", F32, (T, H))
    _check(chan, "chan", F32, (T, H, dim))
    _check(state, "state", F32, (None, H, dim, vdim))
    _check(out, "out", F32, (T, H, vdim))
    R = _check_rows((None, *step_rows[1:]), 0)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_delta_scan_channels", _ptr(qkv), C, G, dim, H, vdim, _ptr(beta), _ptr(chan), _ptr(state), _ptr(row_first),
         _ptr(row_len), _ptr(row_start), _ptr(row_slots), int(bool(writes)), _ptr(out), R, int(slices), _stream())  # fmt: skip


MEMORY_MAX_KEY_DIM = 512  # a lane keeps at most 32 rows of a column of the state beside the normaliser's


def memory_prepare(proj, q_off, k_off, v_off, i_off, f_off, num_heads, dim, vdim, i_bias, f_bias, cap, qkv, i_log, f_log) -> None:
    """What a matrix memory's scan reads, in fp32: qkv [T, 2 H dim + H vdim] = the queries times dim^(-1/2), the keys and
    the values out of proj [T, ld]; i_log = cap tanh((proj[:, i_off + h] + i_bias[h]) / cap) and f_log = logsigmoid(cap
    tanh((proj[:, f_off + h] + f_bias[h]) / cap)), both [T, H]."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H = num_heads
    if min(q_off, k_off, v_off, i_off, f_off) < 0 or max(q_off, k_off) + H * dim > ld or v_off + H * vdim > ld \
            or max(i_off, f_off) + H > ld:  # fmt: skip
        raise KernelError("memory_prepare: columns outside the projection")
    _check(i_bias, "i_bias", F32, (H,))
    _check(f_bias, "f_bias", F32, (H,))
    _check(qkv, "qkv", F32, (T, 2 * H * dim + H * vdim))
    _check(i_log, "i_log", F32, (T, H))
    _check(f_log, "f_log", F32, (T, H))
    call("as_memory_prepare", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, i_off, f_off, H, dim, vdim,
         _ptr(i_bias), _ptr(f_bias), float(cap), _ptr(qkv), _ptr(i_log), _ptr(f_log), T, _stream())  # fmt: skip


def memory_scan(qkv, num_heads, dim, vdim, i_log, f_log, state, norm_state, max_state, step_rows, out, writes=True, slices=0) -> None:
    """A matrix memory with exponential gates over each row's tokens, per head, with a running maximum m (0 at a
    sequence's start): m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T; n' likewise with k;
    out = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6).  state [slots, H, dim, vdim], norm_state [slots, H, dim], max_state
    [slots, H], all fp32; qkv, i_log, f_log as `memory_prepare` left them; out fp32 [T, H, vdim]."""
    _check(qkv, "qkv", F32, (None, None))
    T, C = qkv.shape
    H = num_heads
    if C != 2 * H * dim + H * vdim or dim > MEMORY_MAX_KEY_DIM:
        raise KernelError(f"memory_scan: {C} channels are not {H} x (2 x {dim} + {vdim}), or keys wider than {MEMORY_MAX_KEY_DIM}")
    _check(i_log, "i_log", F32, (T, H))
    _check(f_log, "f_log", F32, (T, H))
    _check(state, "state", F32, (None, H, dim, vdim))
    slots = state.shape[0]
    _check(norm_state, "norm_state", F32, (slots, H, dim))
    _check(max_state, "max_state", F32, (slots, H))
    _check(out, "out", F32, (T, H, vdim))
    R = _check_rows((None, *step_rows[1:]), 0)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_memory_scan", _ptr(qkv), C, dim, H, vdim, _ptr(i_log), _ptr(f_log), _ptr(state), _ptr(norm_state),
         _ptr(max_state), _ptr(row_first), _ptr(row_len), _ptr(row_start), _ptr(row_slots), int(bool(writes)), _ptr(out),
         R, int(slices), _stream())  # fmt: skip


def rglru_gates(u, ra, ra_bias, ri, ri_bias, lam, c, a_out, x_out) -> None:
    """The two gates of a gated linear recurrence, per block of channels (ra, ri [blocks, bw, bw], out x in):
    r = sigmoid(ra u_b + ra_bias), i = sigmoid(ri u_b + ri_bias); a_out = exp(-c r softplus(lam)),
    x_out = sqrt(1 - a^2) i u.  u, a_out, x_out fp32 [T, width]."""
    _check(u, "u", F32, (None, None))
    T, width = u.shape
    _check(ra, "ra", (F32, BF16), (None, None, None))
    blocks, bw, _ = ra.shape
    if blocks * bw != width or ra.shape[2] != bw:
        raise KernelError(f"rglru_gates: {blocks} blocks of {tuple(ra.shape[1:])} do not make {width} channels")
    _check(ri, "ri", ra.dtype, (blocks, bw, bw))
    for name, v in (("ra_bias", ra_bias), ("ri_bias", ri_bias), ("lam", lam)):
        _check(v, name, ra.dtype)
        if v.numel() != width:
            raise KernelError(f"{name} has {v.numel()} entries for {width} channels")
    _check(a_out, "a_out", F32, (T, width))
    _check(x_out, "x_out", F32, (T, width))
    call("as_rglru_gates", _ptr(u), width, blocks, _ptr(ra), _ptr(ra_bias), _ptr(ri), _ptr(ri_bias), _ptr(lam),
         _DT[ra.dtype], float(c), _ptr(a_out), _ptr(x_out), T, _stream())  # fmt: skip


def rglru_scan(a, x, proj, y_off, y_bias, scale, state, step_rows, out, out_off, writes=True) -> None:
    """S = a S + x per channel over each row's tokens (state fp32 [slots, width]; from zero at position 0);
    out[t, out_off + c] = scale * S * gelu_tanh(proj[t, y_off + c] + y_bias[c])."""
    _check(a, "a", F32, (None, None))
    T, width = a.shape
    _check(x, "x", F32, (T, width))
    _check(proj, "proj", (F32, BF16), (T, None))
    _check(out, "out", proj.dtype, (T, None))
    if y_off < 0 or y_off + width > proj.shape[1] or out_off < 0 or out_off + width > out.shape[1]:
        raise KernelError("rglru_scan: columns outside the projection or the output")
    w_dtype = _vector_dtype(proj.dtype, y_bias)
    if y_bias is not None:
        _check(y_bias, "y_bias", w_dtype, (width,))
    _check(state, "state", F32, (None, width))
    R = _check_rows((None, *step_rows[1:]), 0)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_rglru_scan", _ptr(a), _ptr(x), width, _ptr(proj), _DT[proj.dtype], proj.shape[1], y_off, _ptr(y_bias),
         _DT[w_dtype], float(scale), _ptr(state), _ptr(row_first), _ptr(row_len), _ptr(row_start), _ptr(row_slots),
         int(bool(writes)), _ptr(out), out.shape[1], out_off, R, _stream())  # fmt: skip


# ---- experts ------------------------------------------------------------------------------------------

MOE_TILE = 64  # pairs of one expert that a workgroup of the grouped products takes
MOE_MAX_EXPERTS = 1024


class ExpertRoute:
    """Where a step's (token, chosen expert) pairs stand once sorted by expert: what the grouped products read."""

    __slots__ = ("order", "tiles", "counts", "max_tiles", "top", "num_tokens", "pair_weight")

    def __init__(self, num_tokens: int, top: int, experts: int, device):
        pairs = num_tokens * top
        self.max_tiles = -(-pairs // MOE_TILE) + experts
        self.order = torch.empty(max(pairs, 1), dtype=I32, device=device)
        self.tiles = torch.empty((self.max_tiles, 3), dtype=I32, device=device)
        self.counts = torch.empty(1, dtype=I32, device=device)
        self.top, self.num_tokens = top, num_tokens
        self.pair_weight = None  # fp32 [pairs]: what each pair weighs, where a router says (else all weigh alike)


def moe_route_table(token_ids, table, experts: int) -> ExpertRoute:
    """Routes by a table [vocab, top] int32 that names every token id's experts."""
    _check(token_ids, "token_ids", I32, (None,))
    _check(table, "table", I32, (None, None))
    vocab, top = table.shape
    if not 1 <= experts <= MOE_MAX_EXPERTS:
        raise KernelError(f"routing sorts up to {MOE_MAX_EXPERTS} experts, not {experts}")
    route = ExpertRoute(token_ids.shape[0], top, experts, token_ids.device)
    call("as_moe_route_table", _ptr(token_ids), _ptr(table), vocab, top, experts, token_ids.shape[0], _ptr(route.order),
         _ptr(route.tiles), _ptr(route.counts), route.max_tiles, _stream())  # fmt: skip
    return route


def moe_route_sigmoid(h, router, top: int) -> ExpertRoute:
    """Routes by a router's scores: z = router h in fp32, s = sigmoid(z), a token's `top` experts those with the
    largest s, weighing s / (their sum + 1e-20).  h [T, K], router [experts, K] of one dtype.  The route carries
    `pair_weight` fp32 [T * top] for `moe_combine`."""
    return moe_route_scores(h, router, top, "sigmoid")


ROUTER_SCORES = {"sigmoid": 0, "softmax_of_chosen": 1, "softmax": 2}


def moe_route_scores(h, router, top: int, score: str, bias=None, groups: int = 1, keep_groups: int = 1,
                     weight_scale: float = 1.0) -> ExpertRoute:  # fmt: skip
    """Routes by a router's logits z = router h + bias in fp32 (bias fp32 [experts] or None).  score "sigmoid": the
    `top` largest sigmoid(z), weighing s / (their sum + 1e-20); "softmax_of_chosen": the `top` largest z, weighing the
    softmax over those z alone; "softmax": s = softmax(z) over all experts, the `top` largest among the experts of the
    `keep_groups` best of `groups` equal groups of neighbours (a group scores its largest s), weighing s * weight_scale.
    The route carries `pair_weight` fp32 [T * top] for `moe_combine`."""
    _check(h, "h", (F32, BF16), (None, None))
    T, K = h.shape
    _check(router, "router", h.dtype, (None, K))
    experts = router.shape[0]
    if score not in ROUTER_SCORES:
        raise KernelError(f"a router scores by one of {sorted(ROUTER_SCORES)}, not by {score!r}")
    if bias is not None:
        _check(bias, "bias", F32, (experts,))
    if not 1 <= top <= experts <= MOE_MAX_EXPERTS:
        raise KernelError(f"routing chooses up to {MOE_MAX_EXPERTS} experts, not {top} of {experts}")
    if score != "softmax" and (groups, keep_groups, weight_scale) != (1, 1, 1.0):
        raise KernelError("groups of experts and a scale of the weights belong to the score 'softmax'")
    if groups < 1 or experts % groups or not 1 <= keep_groups <= groups or keep_groups * (experts // groups) < top:
        raise KernelError(f"{experts} experts in {groups} groups of which {keep_groups} are kept do not give {top} to choose")
    route = ExpertRoute(T, top, experts, h.device)
    pair_expert = torch.empty(max(T * top, 1), dtype=I32, device=h.device)
    route.pair_weight = torch.empty(max(T * top, 1), dtype=F32, device=h.device)
    call("as_moe_route_scores", _ptr(h), _ptr(router), _ptr(bias), ROUTER_SCORES[score], int(groups), int(keep_groups),
         float(weight_scale), _DT[h.dtype], K, experts, top, T,
         _ptr(pair_expert), _ptr(route.pair_weight), _stream())  # fmt: skip
    call("as_moe_route_table", 0, _ptr(pair_expert), 0, top, experts, T, _ptr(route.order), _ptr(route.tiles),
         _ptr(route.counts), route.max_tiles, _stream())  # fmt: skip
    return route


def moe_gemm(a, w, route: ExpertRoute, out, gated: bool, per_token: bool, activation: str = None, limit: float = 0.0) -> None:
    """The product of every pair's input with its expert's matrix, w [experts, N_w, K].  per_token: a [T, K] holds
    a row per token (all of a token's pairs read it), else a row per pair.  gated: N_w = 2 N, out[p] =
    silu(w[e, :N] a) * (w[e, N:] a), or with limit > 0 the gated activation with limits (`clamped_gate`); else
    out[p] = w[e] a, or relu(w[e] a)^2 with activation "relu2".  out [pairs, N]: a's dtype, or fp32."""
    if limit < 0 or (limit and not gated):
        raise KernelError("moe_gemm: a limit (positive) belongs to a gated product")
    _check(a, "a", (F32, BF16), (None, None))
    K = a.shape[1]
    pairs = route.num_tokens * route.top
    if a.shape[0] != (route.num_tokens if per_token else pairs):
        raise KernelError(f"moe_gemm: {a.shape[0]} input rows for {route.num_tokens} tokens of {route.top} experts")
    _check(w, "w", a.dtype, (None, None, K))
    N = w.shape[1] // 2 if gated else w.shape[1]
    if gated and w.shape[1] % 2:
        raise KernelError("moe_gemm: gate and up rows come in equal numbers")
    _check(out, "out", (a.dtype, F32), (pairs, N))
    if activation not in (None, "relu2") or (gated and activation):
        raise KernelError(f"moe_gemm: activation {activation!r} (None, or 'relu2' on a product without a gate)")
    if (gated or activation) and out.dtype != a.dtype:
        raise KernelError("moe_gemm: the activated product's result has the inputs' dtype")
    call("as_moe_gemm", _ptr(a), _DT[a.dtype], route.top if per_token else 1, _ptr(w), N, K,
         2 if activation else int(bool(gated)),
         _ptr(route.order), _ptr(route.tiles), _ptr(route.counts), route.max_tiles, _ptr(out), _DT[out.dtype], float(limit), _stream())  # fmt: skip


def moe_combine(pair_out, top: int, weight: float, out, pair_weight=None, add=None) -> None:
    """out[t] = sum_j weight * pair_weight[t * top + j] * pair_out[t * top + j] + add[t]; pair_out fp32 [T * top, N];
    pair_weight fp32 [T * top] (None: 1); add [T, N] of out's dtype (None: nothing)."""
    _check(out, "out", (F32, BF16), (None, None))
    T, N = out.shape
    _check(pair_out, "pair_out", F32, (T * top, N))
    if pair_weight is not None:
        _check(pair_weight, "pair_weight", F32, (max(T * top, 1),))
    if add is not None:
        _check(add, "add", out.dtype, (T, N))
    call("as_moe_combine", _ptr(pair_out), top, float(weight), N, _ptr(out), _DT[out.dtype], T, _ptr(pair_weight),
         _ptr(add), _stream())  # fmt: skip


# ---- what a layer does to the stream around its parts ------------------------------------------------------

NORM_MAX_GROUPS = 256
CLAMPED_GATE_ALPHA = 1.702  # the factor inside the sigmoid of the gated activation with limits


def group_norm(x, weight, eps, groups: int, out, delta=None, rows=None, update_x=True) -> None:
    """out[r] = the RMS norm in `groups` equal parts of x[s] (+ delta[s]), times weight; s = rows[r] or r.  x fp32
    [T, n] (receives the sum if update_x), weight fp32 [n], delta and out in the compute dtype."""
    _check(x, "x", F32, (None, None))
    T, n = x.shape
    _check(weight, "weight", F32, (n,))
    _check(out, "out", (F32, BF16), (None, n))
    if delta is not None:
        _check(delta, "delta", out.dtype, (T, n))
    if rows is not None:
        _check(rows, "rows", I32, (out.shape[0],))
    elif out.shape[0] != T:
        raise KernelError("group_norm: one output row per row of the stream")
    if not 1 <= groups <= NORM_MAX_GROUPS or n % groups:
        raise KernelError(f"group_norm: {n} columns do not divide into {groups} groups (at most {NORM_MAX_GROUPS})")
    call("as_group_norm", _ptr(x), _ptr(delta), _ptr(rows), _ptr(weight), float(eps), groups, _ptr(out), _DT[out.dtype],
         out.shape[0], n, int(bool(update_x)), _stream())  # fmt: skip


def group_norm_shift(x, weight, mu, eps, groups: int, step_rows, state, out, writes=True) -> None:
    """The grouped norm of every token's row and a token shift after it: out[t] = h_t + (h' - h_t) * mu with h' the
    normed row of the token before, zeros at a sequence's first token, and for a row's first token what its request's
    slot in `state` [slots, n] fp32 holds; the slot then receives the row's last normed row (unless `writes` is off)."""
    _check(x, "x", F32, (None, None))
    T, n = x.shape
    _check(weight, "weight", F32, (n,))
    _check(mu, "mu", F32, (n,))
    _check(out, "out", (F32, BF16), (T, n))
    _check(state, "state", F32, (None, n))
    _check_rows(step_rows, T)
    tok_row, row_first, row_len, row_start, row_slots = step_rows
    if not 1 <= groups <= NORM_MAX_GROUPS or n % groups:
        raise KernelError(f"group_norm_shift: {n} columns do not divide into {groups} groups (at most {NORM_MAX_GROUPS})")
    call("as_group_norm_shift", _ptr(x), _ptr(weight), _ptr(mu), float(eps), groups, _ptr(tok_row), _ptr(row_first),
         _ptr(row_len), _ptr(row_start), _ptr(row_slots), _ptr(state), _ptr(out), _DT[out.dtype], T, n,
         int(bool(writes)), _stream())  # fmt: skip


def depth_average(x, delta, kept, coef, n: int) -> None:
    """v = x + delta is kept as kept[n]; x = sum_(j < n) coef[j] kept[j] + coef[n] v.  x fp32 [T, w]; delta [T, w] in
    the compute dtype or None; kept fp32 [slots > n, T, w]; coef fp32 [n + 1]."""
    _check(x, "x", F32, (None, None))
    _check(kept, "kept", F32, (None, *x.shape))
    _check(coef, "coef", F32, (n + 1,))
    if not 0 <= n < kept.shape[0]:
        raise KernelError(f"depth_average: result {n} of {kept.shape[0]} kept")
    dtype = F32
    if delta is not None:
        _check(delta, "delta", (F32, BF16), tuple(x.shape))
        dtype = delta.dtype
    call("as_depth_average", _ptr(x), _ptr(delta), _DT[dtype], _ptr(kept), _ptr(coef), n, x.numel(), _stream())


def clamped_gate(gate_up, out, limit: float) -> None:
    """out = g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit); gate_up [T, 2 I]:
    a row's gate values, then its up values."""
    _check(gate_up, "gate_up", (F32, BF16), (None, None))
    T, two_i = gate_up.shape
    if two_i % 2 or not limit > 0:
        raise KernelError("clamped_gate: gate and up come in equal numbers, and the limit is positive")
    _check(out, "out", gate_up.dtype, (T, two_i // 2))
    call("as_clamped_gate", _ptr(gate_up), _ptr(out), _DT[gate_up.dtype], T, two_i // 2, float(limit), CLAMPED_GATE_ALPHA,
         _stream())  # fmt: skip


def gemm_clamped_gate(a, w, out, limit: float, choices=None) -> None:
    """out = clamped_gate(a @ w^T, limit): w [2 I, K] holds the gate rows, then the up rows; out [T, I]."""
    M, K = a.shape
    rows = _rows(w)
    inter = rows.shape[0] // 2
    if a.dtype == BF16 and M and limit > 0 and (_few_rows(M, K, inter, GATED_MAX_K, w=w) or _gated_two_tiles(M, K, w)):
        # few rows: the product that streams the weights applies the activation on its way out
        _check(rows, "w", a.dtype, (2 * inter, K))
        _check(out, "out", a.dtype, (M, inter))
        call("as_gemm_bf16_gated_limited", _ptr(a), _ptr(rows), _wave_ptr(w), _ptr(out), M, inter, K, float(limit),
             CLAMPED_GATE_ALPHA, _stream())  # fmt: skip
        return
    gate_up = torch.empty((M, rows.shape[0]), dtype=a.dtype, device=a.device)
    gemm(a, w, gate_up, choices)
    clamped_gate(gate_up, out, limit)


# ---- linear attention with a fixed decay per head -------------------------------------------------------------

ACTIVATIONS = {None: 0, "silu": 1, "sigmoid": 2}
DECAY_SCAN_MAX_DIM = 512


def decay_scan(proj, q_off, k_off, v_off, num_heads, dim, vdim, activation, k_scale, decay, state, step_rows, out,
               writes=True) -> None:  # fmt: skip
    """S = decay_h S + k v^T, o = S^T q per head and token, in the order of a row's tokens.  q, k [heads, dim] and v
    [heads, vdim] are columns q_off.., k_off.., v_off.. of proj [T, ld] after `activation` (None or "silu"), k also
    times k_scale.  decay fp32 [heads]; state fp32 [slots, heads, dim, vdim]; out fp32 [T, heads, vdim]."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H, D, E = num_heads, dim, vdim
    if activation not in (None, "silu"):
        raise KernelError(f"decay_scan: activation {activation!r} (None or 'silu')")
    if min(H, D, E) < 1 or D > DECAY_SCAN_MAX_DIM or max(q_off + H * D, k_off + H * D, v_off + H * E) > ld or min(q_off, k_off, v_off) < 0:
        raise KernelError(f"decay_scan: {H} heads of {D} and {E} at columns {q_off}, {k_off}, {v_off} of {ld}")
    _check(decay, "decay", F32, (H,))
    _check(state, "state", F32, (None, H, D, E))
    _check(out, "out", F32, (T, H, E))
    R = _check_rows(step_rows, T)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_decay_scan", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, H, D, E, ACTIVATIONS[activation],
         float(k_scale), _ptr(decay), _ptr(state), _ptr(row_first), _ptr(row_len), _ptr(row_start), _ptr(row_slots), R,
         _ptr(out), int(bool(writes)), _stream())  # fmt: skip


DECAY_CHUNKS_MAX_DIM = 128


def decay_chunks(proj, q_off, k_off, v_off, num_heads, dim, vdim, activation, k_scale, decay, state, step_rows, out,
                 writes=True) -> None:  # fmt: skip
    """What `decay_scan` computes, a row's tokens 32 at a time as fp32 products on the matrix cores: with S the state
    before a chunk of n tokens, o_t = decay^(t+1) S^T q_t + sum_(j <= t) decay^(t-j) (q_t . k_j) v_j and the state
    after it decay^n S + sum_j decay^(n-1-j) k_j v_j^T.  Keys of up to DECAY_CHUNKS_MAX_DIM coordinates."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H, D, E = num_heads, dim, vdim
    if activation not in (None, "silu"):
        raise KernelError(f"decay_chunks: activation {activation!r} (None or 'silu')")
    if min(H, D, E) < 1 or D > DECAY_CHUNKS_MAX_DIM or max(q_off + H * D, k_off + H * D, v_off + H * E) > ld or min(q_off, k_off, v_off) < 0:
        raise KernelError(f"decay_chunks: {H} heads of {D} and {E} at columns {q_off}, {k_off}, {v_off} of {ld}")
    _check(decay, "decay", F32, (H,))
    _check(state, "state", F32, (None, H, D, E))
    _check(out, "out", F32, (T, H, E))
    R = _check_rows(step_rows, T)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_decay_chunks", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, H, D, E, ACTIVATIONS[activation],
         float(k_scale), _ptr(decay), _ptr(state), _ptr(row_first), _ptr(row_len), _ptr(row_start), _ptr(row_slots), R,
         _ptr(out), int(bool(writes)), _stream())  # fmt: skip


def decay_step(proj, q_off, k_off, v_off, num_heads, dim, vdim, activation, k_scale, decay, state, step_rows, out,
               writes=True) -> None:  # fmt: skip
    """What `decay_scan` computes for a step in which every row is ONE token (only each row's first token is taken):
    the state is read and written once, in whole lines.  Keys of up to DECAY_CHUNKS_MAX_DIM, values a multiple of 4."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    H, D, E = num_heads, dim, vdim
    if activation not in (None, "silu"):
        raise KernelError(f"decay_step: activation {activation!r} (None or 'silu')")
    if min(H, D, E) < 1 or D > DECAY_CHUNKS_MAX_DIM or E % 4 or max(q_off + H * D, k_off + H * D, v_off + H * E) > ld or min(q_off, k_off, v_off) < 0:
        raise KernelError(f"decay_step: {H} heads of {D} and {E} at columns {q_off}, {k_off}, {v_off} of {ld}")
    _check(decay, "decay", F32, (H,))
    _check(state, "state", F32, (None, H, D, E))
    _check(out, "out", F32, (T, H, E))
    R = _check_rows(step_rows, T)
    _, row_first, row_len, row_start, row_slots = step_rows
    call("as_decay_step", _ptr(proj), _DT[proj.dtype], ld, q_off, k_off, v_off, H, D, E, ACTIVATIONS[activation],
         float(k_scale), _ptr(decay), _ptr(state), _ptr(row_first), _ptr(row_start), _ptr(row_slots), R, _ptr(out),
         int(bool(writes)), _stream())  # fmt: skip


def decay_attention(proj, q_off, k_off, v_off, num_heads, dim, vdim, activation, k_scale, decay, state, step_rows, out,
                    writes=True) -> None:  # fmt: skip
    """What `decay_scan` computes, by whichever kernel suits the step: token by token where every row is one token (a
    decode step: step_rows names no row per token; values in fours through the kernel that moves whole lines) or the keys
    are wider than the chunked kernel takes, else in chunks."""
    if dim > DECAY_CHUNKS_MAX_DIM:
        kernel = decay_scan
    elif step_rows[0] is None:
        kernel = decay_step if vdim % 4 == 0 else decay_scan
    else:
        kernel = decay_chunks
    kernel(proj, q_off, k_off, v_off, num_heads, dim, vdim, activation, k_scale, decay, state, step_rows, out, writes)


def decay_finish(o, groups: int, eps, gain, proj, g_off, gate_activation, out) -> None:
    """out = norm(o) * gain * act(gate): o fp32 [T, n] normed in `groups` equal parts (RMS, eps inside the root),
    gain fp32 [n] or None, the gate columns g_off.. of proj [T, ld], act "sigmoid" or "silu"; out [T, n] proj's dtype."""
    _check(o, "o", F32, (None, None))
    T, n = o.shape
    _check(proj, "proj", (F32, BF16), (T, None))
    if gain is not None:
        _check(gain, "gain", F32, (n,))
    _check(out, "out", proj.dtype, (T, n))
    if gate_activation not in ("silu", "sigmoid") or groups < 1 or n % groups or g_off < 0 or g_off + n > proj.shape[1]:
        raise KernelError(f"decay_finish: {groups} groups of {n}, gate {gate_activation!r} at column {g_off}")
    call("as_decay_finish", _ptr(o), n, groups, float(eps), _ptr(gain), _ptr(proj), _DT[proj.dtype], proj.shape[1], g_off,
         ACTIVATIONS[gate_activation], _ptr(out), T, _stream())  # fmt: skip


# ---- attention through a latent ---------------------------------------------------------------------------------


LATENT_MAX_RANK, LATENT_MAX_HEAD_DIM = 1536, 1024  # what eight tokens' latents, or heads, may fill of a workgroup's LDS


def rows_rms_norm(proj, off, n, gain, eps, out) -> None:
    """out = RMS norm of columns off..off + n of proj [T, ld], times gain fp32 [n]; out [T, n] proj's dtype."""
    _check(proj, "proj", (F32, BF16), (None, None))
    _check(gain, "gain", F32, (n,))
    _check(out, "out", proj.dtype, (proj.shape[0], n))
    if off < 0 or off + n > proj.shape[1]:
        raise KernelError("rows_rms_norm: columns outside the rows")
    call("as_rows_rms_norm", _ptr(proj), _DT[proj.dtype], proj.shape[1], off, n, _ptr(gain), float(eps), _ptr(out),
         proj.shape[0], _stream())  # fmt: skip


def latent_kv_store(proj, off, rank, rot, gain, eps, cos_sin, slots, k_pages, v_pages) -> None:
    """Columns off.. of proj [T, ld]: `rank` of the latent (RMS-normed here, times gain fp32 [rank]) and `rot` of the
    shared key part (turned here by cos_sin [T, rot/2, 2] fp32).  [latent | key part | zeros] goes to the key pages
    [pages, 1, bs, width] at slots[t] (< 0: nowhere), [latent | zeros] to the value pages [pages, 1, width, bs]."""
    _check(proj, "proj", (F32, BF16), (None, None))
    T, ld = proj.shape
    _check(gain, "gain", F32, (rank,))
    _check(slots, "slots", I32, (T,))
    _check(k_pages, "k_pages", proj.dtype, (None, 1, None, None))
    pages, _, bs, width = k_pages.shape
    _check(v_pages, "v_pages", proj.dtype, (pages, 1, width, bs))
    if rot:
        _check(cos_sin, "cos_sin", F32, (T, rot // 2, 2))
    if rank < 1 or rot < 0 or rot % 2 or rank + rot > width or off < 0 or off + rank + rot > ld:
        raise KernelError(f"latent_kv_store: a latent of {rank} and a key part of {rot} in pages of {width}, rows of {ld}")
    call("as_latent_kv_store", _ptr(proj), _DT[proj.dtype], ld, off, rank, rot, _ptr(gain), float(eps), _ptr(cos_sin),
         _ptr(slots), _ptr(k_pages), _ptr(v_pages), bs, width, T, _stream())  # fmt: skip


def latent_q_absorb(q, uk, num_heads, dim, rot, rank, cos_sin, out, uk_t=None) -> None:
    """q [T, heads * (dim + rot)], uk [heads * dim, rank]: out[t, h] = [uk_h^T q_h[:dim] | q_h[dim:] turned by
    cos_sin | zeros]; out [T, heads, width].  uk_t [heads, rank, dim]: the same matrices transposed, with which
    bfloat16 prompts multiply on the matrix cores."""
    _check(q, "q", (F32, BF16), (None, num_heads * (dim + rot)))
    T = q.shape[0]
    _check(uk, "uk", q.dtype, (num_heads * dim, rank))
    if uk_t is not None:
        _check(uk_t, "uk_t", q.dtype, (num_heads, rank, dim))
    _check(out, "out", q.dtype, (T, num_heads, None))
    if rot:
        _check(cos_sin, "cos_sin", F32, (T, rot // 2, 2))
    if rank + rot > out.shape[2] or rot % 2 or dim > LATENT_MAX_HEAD_DIM:
        raise KernelError("latent_q_absorb: the latent and the turned part exceed the output's width, or the heads the kernel's")
    call("as_latent_q_absorb", _ptr(q), _ptr(uk), _ptr(uk_t), _DT[q.dtype], num_heads, dim, rot, rank, _ptr(cos_sin),
         _ptr(out), out.shape[2], T, _stream())  # fmt: skip


def latent_v_expand(heads, uv_t, rank, gate, g_off, out, uv=None) -> None:
    """heads [T, H, width] (the first `rank` coordinates count), uv_t [H, rank, E]: out[t, h E + e] = (sum_r heads[t, h,
    r] uv_t[h, r, e]) * sigmoid(gate[t, g_off + h E + e]); gate [T, ld] or None (no gate); out [T, H * E].  uv [H * E,
    rank]: the same matrices as a checkpoint holds them, with which bfloat16 prompts multiply on the matrix cores."""
    _check(heads, "heads", (F32, BF16), (None, None, None))
    T, H, width = heads.shape
    _check(uv_t, "uv_t", heads.dtype, (H, rank, None))
    E = uv_t.shape[2]
    if uv is not None:
        _check(uv, "uv", heads.dtype, (H * E, rank))
    _check(out, "out", heads.dtype, (T, H * E))
    ld = 0
    if gate is not None:
        _check(gate, "gate", heads.dtype, (T, None))
        ld = gate.shape[1]
        if g_off < 0 or g_off + H * E > ld:
            raise KernelError("latent_v_expand: the gate's columns lie outside its rows")
    if rank > width or rank > LATENT_MAX_RANK:
        raise KernelError("latent_v_expand: the latent is wider than the heads, or than the kernel takes")
    call("as_latent_v_expand", _ptr(heads), _ptr(uv_t), _ptr(uv), _DT[heads.dtype], H, E, rank, width, _ptr(gate), ld,
         g_off, _ptr(out), T, _stream())  # fmt: skip


WIDE_ATTEND_MAX_WIDTH = 2048


def wide_attend(q, k_pages, v_pages, positions, tok_row, block_tables, out, scale, max_context) -> None:
    """Causal attention of every token's heads q [T, H, width] over ONE kv head of any width up to
    WIDE_ATTEND_MAX_WIDTH (k_pages [pages, 1, bs, width], v_pages [pages, 1, width, bs]): for pages wider than the
    paged attention kernels' heads.  positions, tok_row [T] int32 (tok_row None: token t is row t); out like q."""
    _check(q, "q", (F32, BF16), (None, None, None))
    T, H, width = q.shape
    _check(out, "out", q.dtype, (T, H, width))
    _check(k_pages, "k_pages", q.dtype, (None, 1, None, width))
    pages, _, bs, _ = k_pages.shape
    _check(v_pages, "v_pages", q.dtype, (pages, 1, width, bs))
    _check(positions, "positions", I32, (T,))
    if tok_row is not None:
        _check(tok_row, "tok_row", I32, (T,))
    _check(block_tables, "block_tables", I32, (None, None))
    if tok_row is None and block_tables.shape[0] < T:
        raise KernelError(f"attention: {T} tokens that are their own rows need as many block tables")
    if width > WIDE_ATTEND_MAX_WIDTH:
        raise KernelError(f"attention: heads of {width} exceed {WIDE_ATTEND_MAX_WIDTH}")
    if max_context > block_tables.shape[1] * bs:
        raise KernelError("attention: block tables are shorter than the longest context")
    call("as_wide_attend", _ptr(q), _ptr(k_pages), _ptr(v_pages), _DT[q.dtype], _ptr(positions), _ptr(tok_row),
         _ptr(block_tables), block_tables.shape[1], _ptr(out), H, width, bs, float(scale), T, _stream())
