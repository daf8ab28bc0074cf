"""Python face of the HIP kernel library (ctypes, plain C ABI).

Each wrapper checks devices, dtypes, contiguity and shapes on the host, then
passes raw pointers and the current HIP stream. There is no fallback: when the
library cannot be loaded or a tensor is not on the GPU, the call raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p
from typing import Optional, Sequence

import torch

from .csrc.build import ensure_built

PAGE = 64          # tokens per cache page, fixed in csrc/common.h (TA_PAGE)
F32, BF16 = 0, 1


class KernelError(RuntimeError):
    pass


_lib = None


def library():
    """Loads (and on first use builds) the kernel library."""
    global _lib
    if _lib is None:
        path = ensure_built()
        lib = ctypes.CDLL(str(path))
        lib.ta_last_error.restype = c_char_p
        if lib.ta_page_size() != PAGE:
            raise KernelError(f"kernel library pages hold {lib.ta_page_size()} tokens, "
                              f"the Python side expects {PAGE}")
        lib._path = str(path)
        _lib = lib
    return _lib


def library_path() -> str:
    return library()._path


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


def _dev(t: torch.Tensor, name: str, dtype=None, contiguous=True):
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}; kernels run on the GPU only")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous")
    return t


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int):
    if rc != 0:
        raise KernelError(library().ta_last_error().decode())


def _rows2d(t: torch.Tensor, name: str):
    """(rows, row stride) of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name}: expected a 2-D tensor with contiguous rows, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    return t.shape[0], t.stride(0)


def _check_cache_layer(what, kcache, vcache, num_kv_heads, head_dim, value_dim=None):
    """keys [pages, nkv, PAGE, dh]; values transposed inside a page: [pages, nkv, dv, PAGE]
    (dv = dh unless a value width is named)."""
    wk = (kcache.shape[0], num_kv_heads, PAGE, head_dim)
    wv = (kcache.shape[0], num_kv_heads, head_dim if value_dim is None else value_dim, PAGE)
    if tuple(kcache.shape) != wk or tuple(vcache.shape) != wv:
        raise KernelError(f"{what}: cache layer is {tuple(kcache.shape)} / {tuple(vcache.shape)}, "
                          f"expected {wk} / {wv}")


# ------------------------------------------------------------------ embedding
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[tokens[t]] as float32. tokens: int32 [nt]; out: float32 [nt, d]."""
    _dev(table, "table"); _dev(tokens, "tokens", torch.int32); _dev(out, "out", torch.float32)
    vocab, d = table.shape
    nt = tokens.numel()
    if out.shape != (nt, d):
        raise KernelError(f"embed: out is {tuple(out.shape)}, expected {(nt, d)}")
    _check(library().ta_embed(_stream(), _code(table.dtype), _ptr(table), c_int(vocab), c_int(d),
                              _ptr(tokens), c_int(nt), _ptr(out)))
    return out


# ------------------------------------------------------------------ add + norm
def add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                delta: Optional[torch.Tensor] = None, delta_bias: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """v = x[r] + delta[r] + delta_bias; out[i] = rmsnorm(v) * weight.

    Without ``rows`` r = i and, when there is anything to add, v is stored back
    into x (the float32 residual stream). With ``rows`` (int32) only those rows
    are normalised, into out[0..len(rows)), and x is left as it is. A delta that a
    product left in parts ([planes, nt, d]) is added plane by plane, in order.
    """
    _dev(x, "x", torch.float32); _dev(weight, "weight", torch.float32); _dev(out, "out")
    nt, d = x.shape
    if weight.shape != (d,):
        raise KernelError(f"add_rmsnorm: weight is {tuple(weight.shape)}, expected {(d,)}")
    n_out = nt
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        n_out = rows.numel()
    if out.shape != (n_out, d):
        raise KernelError(f"add_rmsnorm: out is {tuple(out.shape)}, expected {(n_out, d)}")
    ddt, planes, plane = F32, 1, 0
    if delta is not None:
        _dev(delta, "delta")
        if delta.dim() == 3 and delta.shape[1:] == x.shape:
            planes, plane = delta.shape[0], nt * d
        elif delta.shape != x.shape:
            raise KernelError(f"add_rmsnorm: delta is {tuple(delta.shape)}, x is {tuple(x.shape)}")
        ddt = _code(delta.dtype)
    if delta_bias is not None:
        _dev(delta_bias, "delta_bias", torch.float32)
        if delta_bias.shape != (d,):
            raise KernelError("add_rmsnorm: delta_bias must have one entry per column")
    store = int(rows is None and (delta is not None or delta_bias is not None))
    _check(library().ta_add_rmsnorm(_stream(), c_int(ddt), c_int(_code(out.dtype)), _ptr(x),
                                    _ptr(delta), _ptr(delta_bias), _ptr(weight), _ptr(rows),
                                    _ptr(out), c_int(n_out), c_int(d), c_float(eps), c_int(store),
                                    c_int(planes), c_longlong(plane)))
    return out


# ------------------------------------------------------------------ rotary + cache write
def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor,
               magnitude: float = 1.0) -> torch.Tensor:
    """out[t, j] = magnitude * (cos a, sin a) with a = float32(positions[t]) * inv_freq[j] in float32."""
    _dev(positions, "positions", torch.int32); _dev(inv_freq, "inv_freq", torch.float32)
    _dev(out, "out", torch.float32)
    nt, half = positions.numel(), inv_freq.numel()
    if tuple(out.shape) != (nt, half, 2):
        raise KernelError(f"rope_table: out is {tuple(out.shape)}, expected {(nt, half, 2)}")
    _check(library().ta_rope_table_scaled(_stream(), _ptr(positions), _ptr(inv_freq), _ptr(out), c_int(nt),
                                          c_int(half), c_float(magnitude)))
    return out


def rope_kv_write(qkv: torch.Tensor, num_q_heads: int, num_kv_heads: int, head_dim: int,
                  angles: Optional[torch.Tensor], interleaved: bool,
                  dest: Optional[torch.Tensor] = None, kcache: Optional[torch.Tensor] = None,
                  vcache: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None):
    """Rotates q and k inside qkv [nt, (nq + 2 nkv) * dh] in place by the angles of
    ``rope_table`` ([nt, dh/2, 2]; None: no rotation) and stores the step's k and v
    into one cache layer (keys [pages, nkv, PAGE, dh], values [pages, nkv, dh, PAGE])
    at dest [nt] (page * PAGE + offset)."""
    _dev(qkv, "qkv")
    nt = qkv.shape[0]
    width = (num_q_heads + 2 * num_kv_heads) * head_dim
    if qkv.shape != (nt, width):
        raise KernelError(f"rope_kv_write: qkv is {tuple(qkv.shape)}, expected {(nt, width)}")
    if angles is not None:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (nt, head_dim // 2, 2):
            raise KernelError(f"rope_kv_write: angles are {tuple(angles.shape)}, expected "
                              f"{(nt, head_dim // 2, 2)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != width:
            raise KernelError("rope_kv_write: bias must hold one entry per qkv column")
    if kcache is not None:
        _dev(kcache, "kcache", qkv.dtype); _dev(vcache, "vcache", qkv.dtype)
        _dev(dest, "dest", torch.int32)
        _check_cache_layer("rope_kv_write", kcache, vcache, num_kv_heads, head_dim)
        if dest.numel() != nt:
            raise KernelError("rope_kv_write: dest must hold one entry per token")
    _check(library().ta_rope_kv_write(_stream(), c_int(_code(qkv.dtype)), _ptr(qkv), _ptr(bias),
                                      _ptr(dest if kcache is not None else None), _ptr(angles),
                                      c_int(1 if interleaved else 0), _ptr(kcache), _ptr(vcache),
                                      c_int(nt), c_int(num_q_heads), c_int(num_kv_heads),
                                      c_int(head_dim)))
    return qkv


# ------------------------------------------------------------------ attention
def attention_generic(q: torch.Tensor, out: torch.Tensor, kcache: torch.Tensor,
                      vcache: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                      pos0: torch.Tensor, max_qlen: int, num_heads: int, num_kv_heads: int,
                      head_dim: int, scale: float, window: Optional[int] = None):
    """Causal attention of each sequence's new tokens over its cached keys.

    q: [nt, >= nh*dh] (a view whose rows may be wider, e.g. the qkv buffer);
    out: [nt, nh*dh]; kcache [pages, nkv, PAGE, dh], vcache [pages, nkv, dh, PAGE];
    block_table: int32 [B, max_blocks]; cu_q: int32 [B+1]; pos0: int32 [B].
    """
    _dev(q, "q", contiguous=False); _dev(out, "out", q.dtype, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * head_dim or out.shape[1] != num_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {head_dim}")
    _dev(kcache, "kcache", q.dtype); _dev(vcache, "vcache", q.dtype)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, head_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    _check(library().ta_attention_generic(
        _stream(), c_int(_code(q.dtype)), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache),
        _ptr(vcache), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0),
        c_int(B), c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim),
        c_float(scale), c_int(window or 0)))
    return out


def attention(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, max_kv_len, num_heads,
              num_kv_heads, head_dim, scale, window=None):
    """Picks the attention kernel for the step's shape and storage type: bfloat16
    with a head size that is a multiple of 32 runs on the matrix cores (one kernel
    for prompts, one for single tokens that slices the keys); everything else, and
    all of float32, runs the vector-ALU kernel."""
    if q.dtype == torch.bfloat16 and head_dim % 32 == 0 and 32 <= head_dim <= 256:
        if max_qlen == 1 and keys_kernel_fits(num_heads, num_kv_heads, head_dim):
            return attention_keys(q, out, kcache, vcache, block_table, cu_q, pos0, max_kv_len,
                                  num_heads, num_kv_heads, head_dim, scale, window)
        return attention_rows(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen,
                              num_heads, num_kv_heads, head_dim, scale, window)
    return attention_generic(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads,
                             num_kv_heads, head_dim, scale, window)


def _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads, num_kv_heads,
                    head_dim):
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * head_dim or out.shape[1] != num_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {head_dim}")
    _dev(kcache, "kcache", torch.bfloat16); _dev(vcache, "vcache", torch.bfloat16)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, head_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    return B, qs, os_


_cu_count = {}


def compute_units(device) -> int:
    """CUs of the device (workgroups that run at once when each fills a CU)."""
    idx = torch.device(device).index or 0
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def rows_kernel(max_qlen: int, num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    """Which of the prompt kernels takes a launch (``through_lds`` of ``attention_rows``), by
    what was measured on MI355X with 32/8, 64/8 and 32/32 heads of 128, 12/4 of 96, 16/2 and 8/8
    of 64 and 8/8 of 32, prompts of 64 to 16,384 tokens, alone and in batches of equal and of
    unequal lengths: 0 below 256 rows; 1 for heads above 128; else 2 (8B shape: 2,048 tokens
    60 us against 79 of kernel 1, 2,304: 70 against 108, 16,384: 2.30 ms against 2.59, eight
    prompts of 128 to 2,000: 118 against 128)."""
    if max_qlen * (num_heads // num_kv_heads) < 256:
        return 0
    return 1 if head_dim > 128 else 2


def attention_rows(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads,
                   num_kv_heads, head_dim, scale, window=None, through_lds=None):
    """Matrix-core attention for prompts: every wave owns 32 (token, head) rows.
    through_lds: 0: operands straight from memory; 1: the four waves of a workgroup share every
    page through LDS (128 rows a workgroup, two workgroups a CU; head sizes up to 192); 2: the
    same with a wave's scores, softmax and output products overlapped by half pages (head sizes
    up to 128); None: ``rows_kernel`` decides."""
    if through_lds is None:
        through_lds = rows_kernel(max_qlen, num_heads, num_kv_heads, head_dim)
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    _check(library().ta_attention_rows_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache),
        _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0), c_int(B),
        c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_float(scale),
        c_int(window or 0), c_int(int(through_lds))))
    return out


_scratch = {}
_scratch_moves = [0]


def scratch_generation() -> int:
    """Grows whenever kernel scratch memory moves (recorded graphs go stale then)."""
    return _scratch_moves[0]


def _scratch_floats(device, n: int) -> torch.Tensor:
    buf = _scratch.get(device)
    if buf is None or buf.numel() < n:
        buf = torch.empty(max(n, 1 << 16), dtype=torch.float32, device=device)
        _scratch[device] = buf
        _scratch_moves[0] += 1
    return buf


# a unit of work of the single-token attention has at least this many pages unless it is a whole
# sequence. The kernel's time is a floor of about 8 us (launch, the chain record -> pages -> LDS
# -> partial rows) plus its bytes; since the merge asks for all of a sequence's partial rows at
# once, runs of two pages beat runs of four (one sequence of 17 pages: 11.3 against 12.7 us)
_KEYS_MIN_PER = 2


def keys_kernel(group: int, head_dim: int) -> int:
    """Which single-token attention kernel serves ``group`` query heads per kv head: 0 and 1
    name the kernels whose four waves bring a unit's pages in together through LDS (head
    sizes up to 192): 0 gives each wave a quarter of a page's keys for up to 16 query heads
    per kv head, 1 lets every wave form the scores of the whole page for up to 32. Otherwise
    4 waves take pages in turn."""
    return (0 if group <= 16 else 1) if head_dim <= 192 else 4


def key_unit_count(batch: int, num_kv_heads: int) -> int:
    """Units of work into which the sequences of a single-token step are cut (a workgroup is
    one unit of one kv head): at least twice the sequences, so that long ones can still be cut
    when the batch alone fills the CUs, rounded up to whole rounds of one workgroup per CU.
    Measured on the 256 CUs of MI355X with 8 kv heads: 256, 512 and 768 workgroups are good and
    the counts between them bad (12 sequences: 240 workgroups 19.8 us, 288 24.2, 384 22.3; 16
    sequences: 256 23.8, 320 26.8, 512 23.9), because the CUs that get one workgroup more set
    the kernel's time. It depends on the batch size alone, so a recorded graph keeps it."""
    cus = 256
    if torch.cuda.is_available():
        cus = compute_units(torch.cuda.current_device())
    per_round = max(1, cus // max(1, num_kv_heads))
    return max(batch, per_round * -(-2 * batch // per_round))


UNIT_INTS = 8      # int32 values in a unit's record, fixed in csrc/common.h (TA_UNIT_INTS)


def plan_key_units(kv_lens: Sequence[int], n_units: int, min_pages: int = 0, tables=None):
    """Cuts sequences of ``kv_lens`` tokens (this step's token included) into at most
    ``n_units`` runs of pages of about equal length, none shorter than ``min_pages`` unless
    it is a whole sequence: a CU can ask only so much of the memory in a given time, so the
    longest run sets the kernel's time. Returns int32 arrays units [n_units, 8] = (sequence,
    first page, pages, the sequence's length, page numbers of the unit's first two pages (from
    ``tables[b]``, the sequence's row of the block table; 0 without), units of the sequence,
    0), spare units holding 0 pages, and seq_units [batch, 2] = (first unit, units); a
    sequence's units follow one another and cover its pages in order. Pure host."""
    import heapq
    import numpy as np
    min_pages = min_pages or _KEYS_MIN_PER
    B = len(kv_lens)
    if n_units < B:
        raise KernelError(f"{n_units} units of work cannot hold {B} sequences")
    pages = [max(1, -(-int(n) // PAGE)) for n in kv_lens]
    count = [1] * B
    heap = [(-pages[b], b) for b in range(B)]
    heapq.heapify(heap)
    spare = n_units - B
    while spare > 0 and heap:
        _, b = heapq.heappop(heap)
        if pages[b] < min_pages * (count[b] + 1):      # another cut would make its runs too short
            continue
        count[b] += 1
        spare -= 1
        heapq.heappush(heap, (-pages[b] / count[b], b))
    cuts = []
    # sequences with the longest runs first: workgroups start in the order of their units, so
    # where there are more units than the CUs hold at once the short ones fill the end
    for b in sorted(range(B), key=lambda b: (-(pages[b] / count[b]), b)):
        base, extra = divmod(pages[b], count[b])
        first = 0
        for i in range(count[b]):
            n = base + (1 if i < extra else 0)
            cuts.append((b, first, n))
            first += n
    return _unit_records(cuts, kv_lens, n_units, tables)


def _unit_records(cuts, kv_lens, n_units, tables):
    import numpy as np
    units = np.zeros((n_units, UNIT_INTS), dtype=np.int32)
    seq = np.zeros((len(kv_lens), 2), dtype=np.int32)
    for u, (b, first, n) in enumerate(cuts):
        if seq[b, 1] == 0:
            seq[b, 0] = u
        seq[b, 1] += 1
        pa = pb = 0
        if tables is not None:
            pa = int(tables[b][first])
            pb = int(tables[b][first + 1]) if n > 1 else pa
        units[u] = (b, first, n, int(kv_lens[b]), pa, pb, 0, 0)
    for u, (b, _, _) in enumerate(cuts):
        units[u, 6] = seq[b, 1]
    return units, seq


def uniform_key_units(kv_lens: Sequence[int], pages_per_unit: int, tables=None):
    """Units of ``pages_per_unit`` pages each (the last of a sequence may be shorter): the
    plain slicing, for tests that want a given cut. Returns (units, seq_units) as above."""
    cuts = []
    for b, n in enumerate(kv_lens):
        pages = max(1, -(-int(n) // PAGE))
        for first in range(0, pages, pages_per_unit):
            cuts.append((b, first, min(pages_per_unit, pages - first)))
    return _unit_records(cuts, kv_lens, len(cuts), tables)


def attention_keys(q, out, kcache, vcache, block_table, cu_q, pos0, max_kv_len, num_heads,
                   num_kv_heads, head_dim, scale, window=None, slices=None, angles=None,
                   interleaved=False, bias=None, dest=None, units=None, seq_units=None):
    """Matrix-core attention for single tokens (sequence b brings row b of ``q``): the
    keys are cut into units of work that workgroups take in parallel, then merged.

    units, seq_units: int32 tensors on the GPU as ``plan_key_units`` lays them out (the step's
    tables carry them). Without them they are planned here from ``pos0``, which waits for the
    GPU; ``slices`` = (pages per unit, ignored, kernel) then asks for a plain cut and names
    the kernel (see ``keys_kernel``).

    Plain: ``q`` holds rotated q heads and the cache already holds the step's keys and
    values. Fused (``dest`` given): ``q`` is the raw [q | k | v] projection; the bias is
    added, q and k are rotated by ``angles`` ([B, dh/2, 2] from ``rope_table``; None: no
    rotation) and the new key and value are stored at ``dest`` before they are read."""
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    if q.shape[0] != B:
        raise KernelError("attention_keys: every sequence must bring exactly one token")
    group = num_heads // num_kv_heads
    waves = keys_kernel(group, head_dim)
    if slices is not None and len(slices) > 2:
        waves = slices[2]
    if units is None:
        lens = [int(p) + 1 for p in pos0.tolist()]
        if max(lens) > block_table.shape[1] * PAGE:
            raise KernelError("attention_keys: a sequence is longer than the block table")
        host_table = block_table.cpu().numpy()
        if slices is not None:
            u, su = uniform_key_units(lens, int(slices[0]), host_table)
        else:
            u, su = plan_key_units(lens, key_unit_count(B, num_kv_heads), tables=host_table)
        units = torch.from_numpy(u).to(q.device)
        seq_units = torch.from_numpy(su).to(q.device)
    _dev(units, "units", torch.int32); _dev(seq_units, "seq_units", torch.int32)
    if units.dim() != 2 or units.shape[1] != UNIT_INTS or tuple(seq_units.shape) != (B, 2) or units.shape[0] < B:
        raise KernelError(f"attention_keys: units {tuple(units.shape)} / {tuple(seq_units.shape)} "
                          f"for {B} sequences")
    n_units = units.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if dest is not None:
        _dev(dest, "dest", torch.int32)
        if dest.numel() != B or q.shape[1] != width:
            raise KernelError("attention_keys: the fused form needs [q | k | v] rows and one "
                              "destination per sequence")
    if angles is not None:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (B, head_dim // 2, 2):
            raise KernelError(f"attention_keys: angles are {tuple(angles.shape)}, expected "
                              f"{(B, head_dim // 2, 2)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != width:
            raise KernelError("attention_keys: bias must hold one entry per qkv column")
    need = library().ta_attention_keys_scratch
    need.restype = c_longlong
    floats = need(c_int(n_units), c_int(num_heads), c_int(head_dim))
    scratch = _scratch_floats(q.device, floats)
    _check(library().ta_attention_keys_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(bias), _ptr(angles), c_int(1 if interleaved else 0),
        _ptr(dest), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(pos0), c_int(B), c_int(num_heads), c_int(num_kv_heads),
        c_int(head_dim), c_float(scale), c_int(window or 0), _ptr(units), _ptr(seq_units),
        c_int(n_units), c_int(waves), _ptr(scratch)))
    return out


def keys_kernel_fits(num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Whether the single-token matrix-core kernels take this geometry. Those that share pages
    through LDS (head sizes up to 192) hold a fixed amount of it whatever the group; the one
    for larger heads merges its four waves through 4 * (64 + rows * head size) floats, which
    have to fit 64 KB."""
    if head_dim % 32 or not 32 <= head_dim <= 256:
        return False
    group = num_heads // max(num_kv_heads, 1)
    if keys_kernel(group, head_dim) != 4:
        return True
    return (4 * 64 + 4 * min(group, 32) * head_dim) * 4 <= 65536


# ------------------------------------------------------------------ SwiGLU
def swiglu(gate_up: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None):
    """out = silu(gate_up[:, :di]) * gate_up[:, di:]."""
    _dev(gate_up, "gate_up"); _dev(out, "out", gate_up.dtype)
    nt, w = gate_up.shape
    if w % 2 or out.shape != (nt, w // 2):
        raise KernelError(f"swiglu: gate_up {tuple(gate_up.shape)} / out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != w:
            raise KernelError("swiglu: bias must hold one entry per gate_up column")
    _check(library().ta_swiglu(_stream(), c_int(_code(gate_up.dtype)), _ptr(gate_up), _ptr(bias),
                               _ptr(out), c_int(nt), c_int(w // 2)))
    return out


# ------------------------------------------------------------------ matrix product (plain)
def gemm_simple(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor,
                bias: Optional[torch.Tensor] = None):
    """out = a @ w.T (+ bias), float32 accumulation in ascending k for every element. a and
    w share a dtype, or a is bfloat16 and w float32 (a matrix that stays as its file stores it)."""
    _dev(a, "a", contiguous=False)
    _dev(w, "w", None if (a.dtype == torch.bfloat16 and w.dtype == torch.float32) else a.dtype,
         contiguous=False)
    _dev(out, "out", contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w"); Mo, ldc = _rows2d(out, "out")
    K = a.shape[1]
    if w.shape[1] != K or Mo != M or out.shape[1] != N:
        raise KernelError(f"gemm: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (N,):
            raise KernelError("gemm: bias must hold one entry per output column")
    _check(library().ta_gemm_simple(_stream(), c_int(_code(a.dtype)), c_int(_code(w.dtype)),
                                    c_int(_code(out.dtype)),
                                    _ptr(a), c_int(lda), _ptr(w), c_int(ldw), _ptr(bias), _ptr(out),
                                    c_int(ldc), c_int(M), c_int(N), c_int(K)))
    return out


class RowScale:
    """Rows of activations that an RMS norm has not scaled yet: ``parts`` [tiles, 16] float32
    holds sums of squares per row (16 columns each), and the product that reads the rows
    multiplies its result by rsqrt(sum / size + eps)."""

    def __init__(self, parts: torch.Tensor, eps: float, size: int):
        self.parts, self.eps, self.size = parts, float(eps), int(size)


class NormFold:
    """What the product in front of an RMS norm needs to take the norm over: the float32
    residual stream ``x`` [m, n] that its result is added to, the norm's weight [n] and eps,
    the buffer ``h`` [m, n] (bfloat16) for the next product's activations, and scratch for
    the sums of squares. ``scale()`` is what the product behind the norm is given."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, h: torch.Tensor,
                 parts: torch.Tensor):
        self.x, self.weight, self.eps, self.h, self.parts = x, weight, float(eps), h, parts

    @staticmethod
    def parts_shape(size: int):
        return (-(-size // 16), 16)

    def scale(self) -> RowScale:
        return RowScale(self.parts, self.eps, self.x.shape[1])


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor], swiglu: bool = False,
                bias: Optional[torch.Tensor] = None, waves: int = 0,
                scale: Optional[RowScale] = None, fold: Optional[NormFold] = None):
    """out = a @ w.T for at most 16 rows of bfloat16 ``a`` (decode steps), float32
    accumulation, out bfloat16 or float32. swiglu: w is [2*n, k] (gate rows, up rows)
    and out [m, n] = silu(a @ gate.T) * (a @ up.T). waves: 4, 8 or 16 waves of a
    workgroup split k; 0 lets the library choose by the weight's shape.

    scale: the rows of ``a`` still lack their norm's factor, which is applied to the
    product. fold: instead of writing ``out``, the product (+ bias) is added to fold.x,
    and fold.h and fold.parts are prepared for the product behind the next norm."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16, contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w")
    K = a.shape[1]
    n_out = N // 2 if swiglu else N
    if w.shape[1] != K or (swiglu and N % 2):
        raise KernelError(f"gemm_skinny: a {tuple(a.shape)} w {tuple(w.shape)}")
    if fold is None:
        _dev(out, "out", contiguous=False)
        Mo, ldc = _rows2d(out, "out")
        if Mo != M or out.shape[1] != n_out:
            raise KernelError(f"gemm_skinny: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
        out_code = _code(out.dtype)
    else:
        ldc, out_code = n_out, F32
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != N:
            raise KernelError("gemm_skinny: bias must hold one entry per row of w")
    if scale is None and fold is None:
        _check(library().ta_gemm_skinny_bf16(_stream(), c_int(out_code), c_int(int(swiglu)),
                                             _ptr(a), c_int(lda), _ptr(w), c_int(ldw), _ptr(bias),
                                             _ptr(out), c_int(ldc), c_int(M), c_int(n_out), c_int(K),
                                             c_int(waves)))
        return out
    sp, n_parts, eps, size = None, 0, 0.0, 0
    if scale is not None:
        _dev(scale.parts, "scale.parts", torch.float32)
        if scale.parts.dim() != 2 or scale.parts.shape[1] != 16 or scale.size != K or \
                scale.parts.shape[0] != -(-K // 16):
            raise KernelError(f"gemm_skinny: partial sums {tuple(scale.parts.shape)} for rows of {K}")
        sp, n_parts, eps, size = scale.parts, scale.parts.shape[0], scale.eps, scale.size
    x = nw = h = op = None
    ldx = ldh = 0
    if fold is not None:
        if swiglu:
            raise KernelError("gemm_skinny: the activation cannot be followed by the residual")
        _dev(fold.x, "fold.x", torch.float32, contiguous=False)
        _dev(fold.h, "fold.h", torch.bfloat16, contiguous=False)
        _dev(fold.weight, "fold.weight", torch.float32); _dev(fold.parts, "fold.parts", torch.float32)
        Mx, ldx = _rows2d(fold.x, "fold.x"); Mh, ldh = _rows2d(fold.h, "fold.h")
        if Mx != M or Mh != M or fold.x.shape[1] != n_out or fold.h.shape[1] != n_out or \
                fold.weight.numel() != n_out or tuple(fold.parts.shape) != NormFold.parts_shape(n_out):
            raise KernelError(f"gemm_skinny: fold of x {tuple(fold.x.shape)} h {tuple(fold.h.shape)} "
                              f"parts {tuple(fold.parts.shape)} behind a product of {M} x {n_out}")
        x, nw, h, op = fold.x, fold.weight, fold.h, fold.parts
    _check(library().ta_gemm_skinny_norm_bf16(
        _stream(), c_int(out_code), c_int(int(swiglu)), _ptr(a), c_int(lda), _ptr(w), c_int(ldw),
        _ptr(bias), _ptr(out) if fold is None else None, c_int(ldc), c_int(M), c_int(n_out), c_int(K),
        c_int(waves), _ptr(sp), c_int(n_parts), c_float(eps), c_int(size), _ptr(x), c_int(ldx),
        _ptr(nw), _ptr(h), c_int(ldh), _ptr(op)))
    return out


SKINNY_MAX_ROWS = 16
MID_MAX_ROWS = 64


def mid_splits(w: torch.Tensor) -> int:
    """Planes in which ``gemm_mid`` leaves a float32 product of this weight (its shape alone
    decides: few column tiles are cut along k among several workgroups)."""
    return int(library().ta_gemm_mid_splits(c_int(w.shape[0]), c_int(w.shape[1])))


def gemm_mid(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False,
             bias: Optional[torch.Tensor] = None):
    """out = a @ w.T for at most 64 rows of bfloat16 ``a``, float32 accumulation. out is
    [m, n] (bfloat16 or float32) or, float32 only, [planes, m, n] whose planes add up to the
    product (``mid_splits`` planes at most; the bias is in plane 0). swiglu: w is [2*n, k]
    (gate rows, up rows) and out [m, n] = silu(a @ gate.T) * (a @ up.T)."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16, contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w")
    K = a.shape[1]
    n_out = N // 2 if swiglu else N
    if w.shape[1] != K or (swiglu and N % 2):
        raise KernelError(f"gemm_mid: a {tuple(a.shape)} w {tuple(w.shape)}")
    planes, plane = 1, 0
    if out.dim() == 3:
        _dev(out, "out", torch.float32)
        planes, plane = out.shape[0], out.stride(0)
        first = out[0]
    else:
        _dev(out, "out", contiguous=False)
        first = out
    Mo, ldc = _rows2d(first, "out")
    if Mo != M or first.shape[1] != n_out:
        raise KernelError(f"gemm_mid: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != N:
            raise KernelError("gemm_mid: bias must hold one entry per row of w")
    _check(library().ta_gemm_mid_bf16(_stream(), c_int(_code(out.dtype)), c_int(int(swiglu)), _ptr(a),
                                      c_int(lda), _ptr(w), c_int(ldw), _ptr(bias), _ptr(out), c_int(ldc),
                                      c_longlong(plane), c_int(M), c_int(n_out), c_int(K), c_int(planes)))
    return out


def mid_takes(rows: int, w: torch.Tensor) -> bool:
    """Shapes for which ``gemm_mid`` is used instead of the vendor library: more rows than the
    few-rows product takes (or a k too long for it), at most 64."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and 0 < rows <= MID_MAX_ROWS
            and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and w.stride(1) == 1
            and w.data_ptr() % 16 == 0 and not skinny_takes(rows, w))


def mid_wins_plain(rows: int, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` beats the vendor library for a plain product in one plane: 17 to 48
    rows against a weight of 65 to 128 column tiles of 64, which it cuts into workgroups of 32
    columns with four quarters of k each (the qkv product of the 8B shape, 6,144 columns: 13.7,
    14.4, 16.7, 17.3 us at 24, 32, 40, 48 rows against 15.6, 15.8, 18.0, 18.0; at 56 and 64 rows
    20.0 against 18.6: every workgroup's reading of all activations then costs more than is
    won; with fewer tiles there are too few workgroups, with more (10,240 or 12,288 columns)
    the library is level or ahead at every row count)."""
    return mid_takes(rows, w) and rows <= 48 and 64 < -(-w.shape[0] // 64) <= 128


def skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Shapes the few-rows product takes."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and 0 < a.shape[0] <= SKINNY_MAX_ROWS and a.shape[1] % 8 == 0
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def skinny_wins(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the few-rows product is at least as fast as the library's for this shape
    (measured on MI355X with weights from 34 MB to 1 GB, k of 4096 to 28672): up to 8
    rows always; up to 16 rows while k is short, because every workgroup reads its part
    of the activations again and that grows with rows times k."""
    if not skinny_ok(a, w):
        return False
    m = a.shape[0]
    return m <= 8 or a.shape[1] <= 4096


def skinny_fits(rows: int, w: torch.Tensor) -> bool:
    """Whether the few-rows product can take ``rows`` rows of bfloat16 activations in a fresh
    workspace buffer against this weight at all (asked before the activations exist)."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and 0 < rows <= SKINNY_MAX_ROWS
            and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and w.stride(1) == 1
            and w.data_ptr() % 16 == 0)


def skinny_takes(rows: int, w: torch.Tensor) -> bool:
    """``skinny_wins`` in the same terms: also at least as fast as the other products."""
    return skinny_fits(rows, w) and (rows <= 8 or w.shape[1] <= 4096)


def skinny_folds(rows: int, w: torch.Tensor) -> bool:
    """Whether the product in front of a norm should be the few-rows one with the norm folded
    in: up to 16 rows whatever k, because the alternatives pay for the norm's own kernel as
    well (down projection of the 8B shape at 16 rows: 28.6 us against 25.8 + 6.0)."""
    return skinny_fits(rows, w)


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor, out: torch.Tensor):
    """out[i] = index of the highest logit of row i (lowest index among equals)."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(out, "out", torch.int32)
    n, ld = _rows2d(logits, "logits")
    if out.numel() != n:
        raise KernelError("argmax: out must hold one entry per row")
    _check(library().ta_argmax(_stream(), _ptr(logits), c_longlong(ld), c_int(n),
                               c_int(logits.shape[1]), _ptr(out)))
    return out


def sample(logits: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor, temperature: float,
           top_k: int, top_p: float):
    """Draws one token per row from softmax(logits / temperature) cut by top_k / top_p."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(out, "out", torch.int32)
    _dev(uniform, "uniform", torch.float32)
    n, ld = _rows2d(logits, "logits")
    if out.numel() != n or uniform.numel() != n:
        raise KernelError("sample: out and uniform must hold one entry per row")
    vocab = logits.shape[1]
    _check(library().ta_sample(_stream(), _ptr(logits), c_longlong(ld), c_int(n), c_int(vocab),
                               c_float(temperature), c_int(min(int(top_k), vocab)),
                               c_float(top_p), _ptr(uniform), _ptr(out)))
    return out


# ------------------------------------------------------------------ random fill
def fill_normal(out: torch.Tensor, seed: int, stream_id: int, mean: float, std: float):
    """out[i] = mean + std * z_i, z_i standard normal, a function of (seed, stream_id, i)."""
    _dev(out, "out")
    _check(library().ta_fill_normal(_stream(), c_int(_code(out.dtype)), _ptr(out),
                                    c_longlong(out.numel()), ctypes.c_ulonglong(seed & (2**64 - 1)),
                                    ctypes.c_ulonglong(stream_id & (2**64 - 1)), c_float(mean),
                                    c_float(std)))
    return out


# ------------------------------------------------------------------ conversion at load
def read_probe(buf: torch.Tensor, workgroups: int, sink: torch.Tensor) -> None:
    """Launches a kernel that only reads ``buf`` (any dtype, contiguous, a multiple of 16
    bytes) with ``workgroups`` workgroups of 256 threads; ``sink`` is 256 int32 that stay
    untouched. For measuring what the memory gives a plain read."""
    _dev(buf, "buf"); _dev(sink, "sink", torch.int32)
    nbytes = buf.numel() * buf.element_size()
    if sink.numel() < 256:
        raise KernelError("read_probe: sink needs 256 entries")
    _check(library().ta_read_probe(_stream(), _ptr(buf), c_longlong(nbytes), c_int(workgroups), _ptr(sink)))


_CONVERT_SRC = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def convert_takes(src: torch.dtype, dst: torch.dtype) -> bool:
    return src in _CONVERT_SRC and dst in (torch.float32, torch.bfloat16)


def convert(src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
    """dst[i] = src[i] in dst's floating type (float32 or bfloat16) from float32, bfloat16 or
    float16: exact when widening, round-to-nearest-even when narrowing. Flat, same count."""
    _dev(src, "src"); _dev(dst, "dst")
    if not convert_takes(src.dtype, dst.dtype):
        raise KernelError(f"convert: {src.dtype} -> {dst.dtype} is not offered")
    if src.numel() != dst.numel():
        raise KernelError(f"convert: {src.numel()} values into {dst.numel()}")
    _check(library().ta_convert(_stream(), c_int(_CONVERT_SRC[src.dtype]), c_int(_code(dst.dtype)),
                                _ptr(src), _ptr(dst), c_longlong(src.numel())))
    return dst


# ------------------------------------------------------------------ gated activations
_GLU_ACTS = {"silu": 0, "gelu_tanh": 1}


def glu(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu",
        bias: Optional[torch.Tensor] = None):
    """out = act(gate_up[:, :di]) * gate_up[:, di:]; act "silu" or "gelu_tanh"."""
    if activation not in _GLU_ACTS:
        raise KernelError(f"glu: unknown activation {activation!r}; known: {sorted(_GLU_ACTS)}")
    _dev(gate_up, "gate_up"); _dev(out, "out", gate_up.dtype)
    nt, w = gate_up.shape
    if w % 2 or out.shape != (nt, w // 2):
        raise KernelError(f"glu: gate_up {tuple(gate_up.shape)} / out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != w:
            raise KernelError("glu: bias must hold one entry per gate_up column")
    _check(library().ta_glu(_stream(), c_int(_code(gate_up.dtype)), c_int(_GLU_ACTS[activation]),
                            _ptr(gate_up), _ptr(bias), _ptr(out), c_int(nt), c_int(w // 2)))
    return out


# ------------------------------------------------------------------ gated residual, token shift
class GatedDelta:
    """What a gated sublayer leaves for the next norm to add to the float32 residual stream:
    x += mult * sigmoid(gate + gate_bias) * (delta + delta_bias). ``delta`` [nt, d] float32 (or
    [planes, nt, d], added in order); ``gate`` [nt, d] float32, the gate's pre-activation, or
    None for no gate."""

    def __init__(self, delta, delta_bias=None, gate=None, gate_bias=None, mult: float = 1.0):
        self.delta, self.delta_bias = delta, delta_bias
        self.gate, self.gate_bias, self.mult = gate, gate_bias, float(mult)

    def applied(self, x: torch.Tensor) -> torch.Tensor:
        """x + this delta as a new tensor (debugging: the engine lets the next norm add it)."""
        d = self.delta.float().sum(0) if self.delta.dim() == 3 else self.delta.float()
        if self.delta_bias is not None:
            d = d + self.delta_bias
        if self.gate is not None:
            g = self.gate if self.gate_bias is None else self.gate + self.gate_bias
            d = d * torch.sigmoid(g)
        return x + self.mult * d


def norm_shift_fuses(d: int) -> bool:
    """Whether ``gated_add_rmsnorm`` takes the token shift of a single-token step over."""
    return d % 4 == 0 and d <= 4096


def gated_add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                      pending: Optional[GatedDelta] = None,
                      rows: Optional[torch.Tensor] = None, shift=None) -> torch.Tensor:
    """v = x[r] + pending (see ``GatedDelta``); out[i] = v / sqrt(mean(v^2) + eps) * weight.
    Without ``rows`` v is stored back into x; with ``rows`` (int32) only those rows are
    normalised and x is left as it is.

    shift = (mu [d], state [slots, d] float32, slots int32 [nt], shifted [nt, d]): for a step
    in which every sequence brings one token (row i belongs to slots[i]) the token shift runs
    behind the norm in the same kernel: shifted[i] = out[i] + (state[slots[i]] - out[i]) * mu,
    and the state row takes out[i]. Only where ``norm_shift_fuses(d)``."""
    _dev(x, "x", torch.float32); _dev(weight, "weight", torch.float32); _dev(out, "out")
    nt, d = x.shape
    if weight.shape != (d,):
        raise KernelError(f"gated_add_rmsnorm: weight is {tuple(weight.shape)}, expected {(d,)}")
    n_out = nt
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        n_out = rows.numel()
    if out.shape != (n_out, d):
        raise KernelError(f"gated_add_rmsnorm: out is {tuple(out.shape)}, expected {(n_out, d)}")
    delta = dbias = gate = gbias = None
    planes, plane, mult = 1, 0, 1.0
    if pending is not None:
        delta, dbias, gate, gbias, mult = (pending.delta, pending.delta_bias, pending.gate,
                                           pending.gate_bias, pending.mult)
        _dev(delta, "delta", torch.float32)
        if delta.dim() == 3 and delta.shape[1:] == x.shape:
            planes, plane = delta.shape[0], nt * d
        elif delta.shape != x.shape:
            raise KernelError(f"gated_add_rmsnorm: delta is {tuple(delta.shape)}, x {tuple(x.shape)}")
        for t, n in ((dbias, "delta_bias"), (gbias, "gate_bias")):
            if t is not None:
                _dev(t, n, torch.float32)
                if t.shape != (d,):
                    raise KernelError(f"gated_add_rmsnorm: {n} must have one entry per column")
        if gate is not None:
            _dev(gate, "gate", torch.float32)
            if gate.shape != x.shape:
                raise KernelError(f"gated_add_rmsnorm: gate is {tuple(gate.shape)}, x {tuple(x.shape)}")
    if shift is not None:
        mu, state, slots, shifted = shift
        _dev(mu, "mu", torch.float32); _dev(state, "state", torch.float32)
        _dev(slots, "slots", torch.int32); _dev(shifted, "shifted", out.dtype)
        if rows is not None or not norm_shift_fuses(d) or mu.shape != (d,) or state.dim() != 2 \
                or state.shape[1] != d or slots.numel() != nt or shifted.shape != (nt, d):
            raise KernelError(f"gated_add_rmsnorm: the token shift cannot be taken over for rows of {d} "
                              f"(mu {tuple(mu.shape)}, state {tuple(state.shape)}, {slots.numel()} slots)")
        _check(library().ta_gated_add_rmsnorm_shift(
            _stream(), c_int(_code(out.dtype)), _ptr(x), _ptr(delta), c_int(planes), c_longlong(plane),
            _ptr(dbias), _ptr(gate), _ptr(gbias), c_float(mult), _ptr(weight), _ptr(out), c_int(n_out),
            c_int(d), c_float(eps), _ptr(mu), _ptr(state), _ptr(slots), _ptr(shifted)))
        return out
    _check(library().ta_gated_add_rmsnorm(
        _stream(), c_int(_code(out.dtype)), _ptr(x), _ptr(delta), c_int(planes), c_longlong(plane),
        _ptr(dbias), _ptr(gate), _ptr(gbias), c_float(mult), _ptr(weight), _ptr(rows), _ptr(out),
        c_int(n_out), c_int(d), c_float(eps), c_int(int(rows is None))))
    return out


def _step_tables(cu_q, slots, nt, what):
    _dev(cu_q, "cu_q", torch.int32); _dev(slots, "slots", torch.int32)
    batch = slots.numel()
    if cu_q.numel() != batch + 1 or batch < 1 or nt < batch:
        raise KernelError(f"{what}: cu_q / slots disagree about the batch ({cu_q.numel()} / {batch}, "
                          f"{nt} tokens)")
    return batch


def token_shift(h: torch.Tensor, out: torch.Tensor, mu: torch.Tensor, state: torch.Tensor,
                cu_q: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """out[t] = h[t] + (h[t-1] - h[t]) * mu inside each sequence; the row before a sequence's
    first token of the step comes from ``state`` [slots, d] (float32), which then takes the
    sequence's last row of h."""
    _dev(h, "h"); _dev(out, "out", h.dtype); _dev(mu, "mu", torch.float32)
    _dev(state, "state", torch.float32)
    nt, d = h.shape
    batch = _step_tables(cu_q, slots, nt, "token_shift")
    if out.shape != h.shape or mu.shape != (d,) or state.dim() != 2 or state.shape[1] != d:
        raise KernelError(f"token_shift: h {tuple(h.shape)} out {tuple(out.shape)} mu {tuple(mu.shape)} "
                          f"state {tuple(state.shape)}")
    _check(library().ta_token_shift(_stream(), c_int(_code(h.dtype)), _ptr(h), _ptr(out), _ptr(mu),
                                    _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt), c_int(d)))
    return out


def pair_embed_add(x: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor, last_token: torch.Tensor,
                   cu_q: torch.Tensor, pos0: torch.Tensor, slots: torch.Tensor, buckets: int,
                   mul_prev: int, mul_cur: int) -> torch.Tensor:
    """x[t] += table[(previous token * mul_prev + token * mul_cur) % buckets], and
    table[buckets] for a sequence's first token. ``last_token`` [slots] int32 holds every
    sequence's last token between steps."""
    _dev(x, "x", torch.float32); _dev(table, "table"); _dev(tokens, "tokens", torch.int32)
    _dev(last_token, "last_token", torch.int32); _dev(pos0, "pos0", torch.int32)
    nt, d = x.shape
    batch = _step_tables(cu_q, slots, nt, "pair_embed_add")
    if table.shape != (buckets + 1, d) or tokens.numel() != nt or pos0.numel() != batch:
        raise KernelError(f"pair_embed_add: table {tuple(table.shape)} for {buckets} buckets of {d}, "
                          f"{tokens.numel()} tokens for {nt} rows")
    _check(library().ta_pair_embed_add(_stream(), c_int(_code(table.dtype)), _ptr(x), _ptr(table),
                                       _ptr(tokens), _ptr(last_token), _ptr(cu_q), _ptr(pos0), _ptr(slots),
                                       c_int(batch), c_int(nt), c_int(d), c_int(buckets),
                                       c_longlong(mul_prev), c_longlong(mul_cur)))
    return x


def scale_(t: torch.Tensor, s: float) -> torch.Tensor:
    """t *= s in place (float32)."""
    _dev(t, "t", torch.float32)
    _check(library().ta_scale_f32(_stream(), _ptr(t), c_longlong(t.numel()), c_float(s)))
    return t


# ------------------------------------------------------------------ attention with a value width of its own
def qk_prepare(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
               eps: float, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
               angles: Optional[torch.Tensor], rot: int, mix: Optional[torch.Tensor] = None,
               v_first: Optional[torch.Tensor] = None, v_keep: Optional[torch.Tensor] = None,
               dest: Optional[torch.Tensor] = None, kcache: Optional[torch.Tensor] = None,
               vcache: Optional[torch.Tensor] = None, per_head: bool = False,
               k_inplace: bool = False) -> torch.Tensor:
    """On rows [q | k | v] of ``qkv`` (nh*dk, nkv*dk, nkv*dv columns): RMS norm of q and of k
    over all their heads at once (weights given: else none; ``per_head``: every head on its own,
    the weights then have the head's width and serve all heads), rotation of the first ``rot``
    coordinates of every head by ``angles`` [nt, rot/2, 2], v <- (1 - mix) v + mix v_first,
    q written back in place, k and v stored at ``dest`` into the cache layer. ``v_keep``
    receives the values before mixing. The cache's value rows may be wider than the values
    (vcache [pages, nkv, dvs, PAGE], dvs >= value_dim): the rest of a token's column is zeroed.
    ``k_inplace`` (no ``dest``): the keys are written back into their rows as the queries are."""
    _dev(qkv, "qkv", contiguous=False)
    nt, stride = _rows2d(qkv, "qkv")
    nq, nk, nv = num_heads * key_dim, num_kv_heads * key_dim, num_kv_heads * value_dim
    if qkv.shape[1] != nq + nk + nv:
        raise KernelError(f"qk_prepare: rows of {qkv.shape[1]}, expected {nq + nk + nv}")
    normed = q_weight is not None
    if normed:
        _dev(q_weight, "q_weight", torch.float32); _dev(k_weight, "k_weight", torch.float32)
        want = ((key_dim,), (key_dim,)) if per_head else ((nq,), (nk,))
        if (tuple(q_weight.shape), tuple(k_weight.shape)) != want:
            raise KernelError(f"qk_prepare: norm weights are {tuple(q_weight.shape)} / {tuple(k_weight.shape)}, "
                              f"expected {want[0]} / {want[1]}")
    if k_inplace and dest is not None:
        raise KernelError("qk_prepare: the keys go back in place or to the cache, not both")
    if rot:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (nt, rot // 2, 2):
            raise KernelError(f"qk_prepare: angles are {tuple(angles.shape)}, expected {(nt, rot // 2, 2)}")
    else:
        angles = None
    if (mix is None) != (v_first is None):
        raise KernelError("qk_prepare: mix and v_first go together")
    if mix is not None:
        _dev(mix, "mix", torch.float32); _dev(v_first, "v_first", qkv.dtype)
        if mix.numel() != 1 or v_first.shape != (nt, nv):
            raise KernelError(f"qk_prepare: mix {tuple(mix.shape)} / v_first {tuple(v_first.shape)}")
    if v_keep is not None:
        _dev(v_keep, "v_keep", qkv.dtype)
        if v_keep.shape != (nt, nv):
            raise KernelError(f"qk_prepare: v_keep is {tuple(v_keep.shape)}, expected {(nt, nv)}")
    if dest is not None:
        _dev(dest, "dest", torch.int32); _dev(kcache, "kcache", qkv.dtype); _dev(vcache, "vcache", qkv.dtype)
        store_dim = vcache.shape[2] if vcache.dim() == 4 else -1
        if store_dim < value_dim:
            raise KernelError(f"qk_prepare: cache value rows of {store_dim} cannot hold values of {value_dim}")
        _check_cache_layer("qk_prepare", kcache, vcache, num_kv_heads, key_dim, store_dim)
        if dest.numel() != nt:
            raise KernelError("qk_prepare: dest must hold one entry per token")
    _check(library().ta_qk_prepare(
        _stream(), c_int(_code(qkv.dtype)), _ptr(qkv), c_int(stride), _ptr(q_weight), _ptr(k_weight),
        c_float(eps), c_int(2 if normed and per_head else int(normed)), _ptr(angles), c_int(rot), _ptr(mix), _ptr(v_first), _ptr(v_keep),
        _ptr(dest), _ptr(kcache if dest is not None else None), _ptr(vcache if dest is not None else None),
        c_int(nt), c_int(num_heads), c_int(num_kv_heads), c_int(key_dim), c_int(value_dim),
        c_int(store_dim if dest is not None else value_dim), c_int(int(k_inplace))))
    return qkv


def attention_generic_dv(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads,
                         num_kv_heads, key_dim, value_dim, scale, window=None):
    """``attention_generic`` for values of another width than the keys: q [nt, >= nh*dk],
    out [nt, nh*dv], kcache [pages, nkv, PAGE, dk], vcache [pages, nkv, dv, PAGE]."""
    _dev(q, "q", contiguous=False); _dev(out, "out", q.dtype, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * key_dim or out.shape[1] != num_heads * value_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {key_dim} / {value_dim}")
    _dev(kcache, "kcache", q.dtype); _dev(vcache, "vcache", q.dtype)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, key_dim, value_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    _check(library().ta_attention_generic_dv(
        _stream(), c_int(_code(q.dtype)), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache),
        _ptr(vcache), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0),
        c_int(B), c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(key_dim),
        c_int(value_dim), c_float(scale), c_int(window or 0)))
    return out


# ------------------------------------------------------------------ recurrent mixers
def _wcode(w: torch.Tensor, act: torch.dtype, what: str) -> int:
    if w.dtype == act or (act == torch.bfloat16 and w.dtype == torch.float32):
        return _code(w.dtype)
    raise KernelError(f"{what}: activations are {act}, weights {w.dtype}")


def rglru_gates(yx: torch.Tensor, channels: int, x_bias, taps, conv_bias, conv_state, gates_w, gates_b,
                lam, decay_scale: float, cu_q, slots, a_out: torch.Tensor, b_out: torch.Tensor):
    """Decay a_t and input term of the gated diagonal recurrence for every token of the step.
    yx [nt, 2C]: the y branch, then the x branch (before their biases). taps [C, K], conv_state
    [slots, K-1, C]; gates_w [2*blocks, bs, bs] (recurrence-gate blocks, then input-gate blocks),
    gates_b [2*blocks, bs]; a_out, b_out [nt, C] float32."""
    _dev(yx, "yx", contiguous=False)
    nt, stride = _rows2d(yx, "yx")
    C = channels
    batch = _step_tables(cu_q, slots, nt, "rglru_gates")
    for t, n in ((x_bias, "x_bias"), (taps, "taps"), (conv_bias, "conv_bias"), (conv_state, "conv_state"),
                 (gates_b, "gates_b"), (lam, "lam"), (a_out, "a_out"), (b_out, "b_out")):
        _dev(t, n, torch.float32)
    _dev(gates_w, "gates_w")
    K = taps.shape[1]
    nb2, bs = gates_w.shape[0], gates_w.shape[1]
    if yx.shape[1] != 2 * C or taps.shape != (C, K) or x_bias.shape != (C,) or conv_bias.shape != (C,) \
            or lam.shape != (C,) or nb2 % 2 or (nb2 // 2) * bs != C or gates_w.shape != (nb2, bs, bs) \
            or gates_b.shape != (nb2, bs) or conv_state.dim() != 3 or conv_state.shape[1:] != (K - 1, C) \
            or a_out.shape != (nt, C) or b_out.shape != (nt, C):
        raise KernelError(f"rglru_gates: shapes do not fit {C} channels: yx {tuple(yx.shape)} taps "
                          f"{tuple(taps.shape)} gates {tuple(gates_w.shape)} state {tuple(conv_state.shape)}")
    _check(library().ta_rglru_gates(
        _stream(), c_int(_code(yx.dtype)), c_int(_wcode(gates_w, yx.dtype, "rglru_gates")), _ptr(yx),
        c_int(stride), c_int(C), _ptr(x_bias), _ptr(taps), _ptr(conv_bias), c_int(K), _ptr(conv_state),
        _ptr(gates_w), _ptr(gates_b), _ptr(lam), c_float(decay_scale), _ptr(cu_q), _ptr(slots),
        c_int(batch), c_int(nt), c_int(C), c_int(nb2 // 2), _ptr(a_out), _ptr(b_out)))


RGLRU_LIBRARY_ROWS = 256      # from this many tokens on a bfloat16 step's gates go to the matrix cores


def rglru_gates_split(yx: torch.Tensor, channels: int, x_bias, taps, conv_bias, conv_state, gates_w,
                      gates_b, lam, decay_scale: float, cu_q, slots, a_out, b_out, ws) -> None:
    """``rglru_gates`` for long steps with bfloat16 weights: u is formed in float32 and split
    into two bfloat16 numbers whose sum is u to 16 bits of mantissa; the library multiplies both
    by the gates' blocks with float32 sums (one batched product per gate over the blocks), and
    the two products are added before the sigmoid. ``ws``: the step's workspace."""
    _dev(yx, "yx", contiguous=False)
    nt, stride = _rows2d(yx, "yx")
    C = channels
    batch = _step_tables(cu_q, slots, nt, "rglru_gates_split")
    _dev(gates_w, "gates_w", torch.bfloat16)
    nb, bs, K = gates_w.shape[0] // 2, gates_w.shape[1], taps.shape[1]
    if yx.shape[1] != 2 * C or nb * bs != C or gates_w.shape != (2 * nb, bs, bs) or nt > 65535:
        raise KernelError(f"rglru_gates_split: shapes do not fit {C} channels / {nt} tokens")
    u = ws.take("recurrence.u", (nt, C), torch.float32)
    halves = ws.take("recurrence.u_split", (2, nt, C), torch.bfloat16)
    _check(library().ta_rglru_conv_split(
        _stream(), c_int(_code(yx.dtype)), _ptr(yx), c_int(stride), c_int(C), _ptr(x_bias), _ptr(taps),
        _ptr(conv_bias), c_int(K), _ptr(conv_state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt),
        c_int(C), _ptr(u), _ptr(halves[0]), _ptr(halves[1])))
    g = ws.take("recurrence.gates", (2, nb, 2 * nt, bs), torch.float32)
    lhs = halves.view(2 * nt, nb, bs).transpose(0, 1)                 # [nb, 2 nt, bs]: hi rows, then lo rows
    for gate in range(2):
        torch.bmm(lhs, gates_w[gate * nb:(gate + 1) * nb].transpose(1, 2), out_dtype=torch.float32, out=g[gate])
    _check(library().ta_rglru_gates_finish(_stream(), _ptr(g), _ptr(u), _ptr(gates_b), _ptr(lam),
                                           c_float(decay_scale), c_int(nt), c_int(C), c_int(nb),
                                           _ptr(a_out), _ptr(b_out)))


def rglru_scan(yx: torch.Tensor, channels: int, y_bias, x_bias, a_in, b_in, state, conv_state, cu_q,
               slots, out: torch.Tensor, max_qlen: Optional[int] = None,
               scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S_t = a_t S_{t-1} + b_t along every sequence; out_t = S_t * gelu_tanh(y_t + y_bias).
    ``state`` [slots, C] and ``conv_state`` [slots, K-1, C] (float32) are read and left as the
    step's last token leaves them. max_qlen: the most tokens a sequence brings (None: one
    thread walks each channel whatever the length); above 64 the sequences are cut into
    segments that are scanned side by side, which overwrites a_in and b_in and needs
    ``scratch`` [batch, C] float32."""
    _dev(yx, "yx", contiguous=False); _dev(out, "out", yx.dtype)
    nt, stride = _rows2d(yx, "yx")
    C = channels
    batch = _step_tables(cu_q, slots, nt, "rglru_scan")
    for t, n in ((y_bias, "y_bias"), (x_bias, "x_bias"), (a_in, "a_in"), (b_in, "b_in"), (state, "state"),
                 (conv_state, "conv_state")):
        _dev(t, n, torch.float32)
    if yx.shape[1] != 2 * C or out.shape != (nt, C) or a_in.shape != (nt, C) or b_in.shape != (nt, C) \
            or state.dim() != 2 or state.shape[1] != C or conv_state.dim() != 3 or conv_state.shape[2] != C \
            or conv_state.shape[0] != state.shape[0]:
        raise KernelError(f"rglru_scan: shapes do not fit {C} channels")
    if max_qlen is None or scratch is None:
        max_qlen = 1
    else:
        _dev(scratch, "scratch", torch.float32)
        if scratch.shape != (batch, C):
            raise KernelError(f"rglru_scan: scratch is {tuple(scratch.shape)}, expected {(batch, C)}")
    _check(library().ta_rglru_scan(
        _stream(), c_int(_code(yx.dtype)), _ptr(yx), c_int(stride), c_int(C), _ptr(y_bias), _ptr(x_bias),
        _ptr(a_in), _ptr(b_in), _ptr(state), _ptr(conv_state), c_int(conv_state.shape[1] + 1), _ptr(cu_q),
        _ptr(slots), c_int(batch), c_int(max_qlen), c_int(C), _ptr(scratch), _ptr(out)))
    return out


def gla_row_parts(key_dim: int) -> int:
    """Planes in which ``gla_recurrent`` leaves its readout (one per group of key channels that a
    workgroup owns); ``gla_out`` adds them."""
    return int(library().ta_gla_row_parts(c_int(key_dim)))


def gla_recurrent(proj: torch.Tensor, heads: int, key_dim: int, value_dim: int, rank: int, a2, a2_bias,
                  tau: float, state: torch.Tensor, cu_q, slots, o_out: torch.Tensor,
                  alpha: torch.Tensor) -> torch.Tensor:
    """Gated linear attention along every sequence. proj [nt, 2*H*dk + 2*H*dv + rank]: q, k, v,
    the output gate and the low-rank decay input, in that order. Per head S <- diag(alpha) S +
    k v^T with alpha = sigmoid(a2 @ low + a2_bias)^(1/tau), o = S^T (q / sqrt(dk)). ``state``
    [slots, H, dk, dv] float32; ``alpha`` [nt, H*dk] float32 scratch that receives the decays;
    o_out [gla_row_parts(dk), nt, H, dv] float32 planes that add up to the readout."""
    _dev(proj, "proj", contiguous=False)
    nt, stride = _rows2d(proj, "proj")
    H, dk, dv = heads, key_dim, value_dim
    batch = _step_tables(cu_q, slots, nt, "gla_recurrent")
    _dev(a2, "a2"); _dev(a2_bias, "a2_bias", torch.float32); _dev(state, "state", torch.float32)
    _dev(o_out, "o_out", torch.float32); _dev(alpha, "alpha", torch.float32)
    if proj.shape[1] != 2 * H * dk + 2 * H * dv + rank or a2.shape != (H * dk, rank) \
            or a2_bias.shape != (H * dk,) or state.dim() != 4 or state.shape[1:] != (H, dk, dv) \
            or o_out.shape != (gla_row_parts(dk), nt, H, dv) or alpha.shape != (nt, H * dk):
        raise KernelError(f"gla_recurrent: shapes do not fit {H} heads of {dk} / {dv}, rank {rank}: "
                          f"proj {tuple(proj.shape)} a2 {tuple(a2.shape)} state {tuple(state.shape)} "
                          f"o_out {tuple(o_out.shape)} alpha {tuple(alpha.shape)}")
    _check(library().ta_gla_recurrent(
        _stream(), c_int(_code(proj.dtype)), c_int(_wcode(a2, proj.dtype, "gla_recurrent")), _ptr(proj),
        c_int(stride), c_int(0), c_int(H * dk), c_int(2 * H * dk), c_int(2 * H * dk + 2 * H * dv),
        c_int(rank), _ptr(a2), _ptr(a2_bias), c_float(1.0 / tau), c_float(float(dk) ** -0.5), _ptr(alpha),
        _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt), c_int(H), c_int(dk), c_int(dv),
        _ptr(o_out)))
    return o_out


def gla_out(o: torch.Tensor, proj: torch.Tensor, heads: int, key_dim: int, value_dim: int, weight,
            eps: float, out: torch.Tensor) -> torch.Tensor:
    """out = rms_norm(o per head over dv) * weight * silu(gate), o the sum of the planes that
    ``gla_recurrent`` left, the gate being the fourth part of the rows of ``proj``."""
    _dev(o, "o", torch.float32); _dev(proj, "proj", contiguous=False); _dev(out, "out", proj.dtype)
    _dev(weight, "weight", torch.float32)
    nt, stride = _rows2d(proj, "proj")
    H, dk, dv = heads, key_dim, value_dim
    if o.dim() != 4 or o.shape[1:] != (nt, H, dv) or out.shape != (nt, H * dv) or weight.shape != (dv,) \
            or proj.shape[1] < 2 * H * dk + 2 * H * dv:
        raise KernelError(f"gla_out: o {tuple(o.shape)} out {tuple(out.shape)} weight {tuple(weight.shape)}")
    _check(library().ta_gla_out(_stream(), c_int(_code(proj.dtype)), _ptr(o), c_int(o.shape[0]), _ptr(proj),
                                c_int(stride), c_int(2 * H * dk + H * dv), _ptr(weight), c_float(eps),
                                c_int(nt), c_int(H), c_int(dv), _ptr(out)))
    return out


# ------------------------------------------------------------------ results normed before they join the stream
def postnorm_add(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float,
                 xcast: Optional[torch.Tensor] = None, next_weight: Optional[torch.Tensor] = None,
                 next_eps: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += rms_norm(delta, eps) * weight, in float32 and in place. delta [nt, d] or
    [planes, nt, d] float32 (planes added in order). ``xcast`` receives the new rows in its own
    type; ``out`` = rms_norm(new x, next_eps) * next_weight (the stream's next norm, done in
    the same pass). xcast and out share a type."""
    _dev(x, "x", torch.float32); _dev(delta, "delta", torch.float32); _dev(weight, "weight", torch.float32)
    nt, d = x.shape
    planes, plane = 1, 0
    if delta.dim() == 3 and delta.shape[1:] == x.shape:
        planes, plane = delta.shape[0], nt * d
    elif delta.shape != x.shape:
        raise KernelError(f"postnorm_add: delta is {tuple(delta.shape)}, x is {tuple(x.shape)}")
    if weight.shape != (d,):
        raise KernelError(f"postnorm_add: weight is {tuple(weight.shape)}, expected {(d,)}")
    code = None
    for t, n in ((xcast, "xcast"), (out, "out")):
        if t is not None:
            _dev(t, n)
            if t.shape != x.shape or (code is not None and _code(t.dtype) != code):
                raise KernelError(f"postnorm_add: {n} is {tuple(t.shape)} {t.dtype}")
            code = _code(t.dtype)
    if (out is None) != (next_weight is None):
        raise KernelError("postnorm_add: next_weight and out go together")
    if next_weight is not None:
        _dev(next_weight, "next_weight", torch.float32)
        if next_weight.shape != (d,):
            raise KernelError("postnorm_add: next_weight must have one entry per column")
    _check(library().ta_postnorm_add(_stream(), c_int(F32 if code is None else code), _ptr(x), _ptr(delta),
                                     c_int(planes), c_longlong(plane), _ptr(weight), c_float(eps), _ptr(xcast),
                                     _ptr(next_weight), c_float(next_eps), _ptr(out), c_int(nt), c_int(d)))
    return x


_ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "relu2": 2, "silu": 3}


def activation(x: torch.Tensor, out: torch.Tensor, kind: str, side: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(x) (* side), act "gelu" (erf), "gelu_tanh", "relu2" (relu squared) or "silu";
    x, out [nt, n] with contiguous rows (row strides may differ); side float32 [nt, n] likewise."""
    if kind not in _ACTIVATIONS:
        raise KernelError(f"activation: unknown kind {kind!r}; known: {sorted(_ACTIVATIONS)}")
    _dev(x, "x", contiguous=False); _dev(out, "out", x.dtype, contiguous=False)
    nt, xs = _rows2d(x, "x")
    no, os_ = _rows2d(out, "out")
    ss = 0
    if out.shape != x.shape:
        raise KernelError(f"activation: x {tuple(x.shape)} / out {tuple(out.shape)}")
    if side is not None:
        _dev(side, "side", torch.float32, contiguous=False)
        ns, ss = _rows2d(side, "side")
        if side.shape != x.shape:
            raise KernelError(f"activation: side is {tuple(side.shape)}, x {tuple(x.shape)}")
    _check(library().ta_activation(_stream(), c_int(_code(x.dtype)), c_int(_ACTIVATIONS[kind]), _ptr(x), c_int(xs),
                                   _ptr(out), c_int(os_), _ptr(side), c_int(ss), c_int(nt), c_int(x.shape[1])))
    return out


def token_shift_multi(h: torch.Tensor, out: torch.Tensor, mu: torch.Tensor, state: torch.Tensor,
                      cu_q: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """``token_shift`` with several weights at once: mu [n, d], out [n, nt, d]; out[s, t] = h[t] +
    (h[t-1] - h[t]) * mu[s]. The state row of a sequence is read and replaced once."""
    _dev(h, "h"); _dev(out, "out", h.dtype); _dev(mu, "mu", torch.float32); _dev(state, "state", torch.float32)
    nt, d = h.shape
    batch = _step_tables(cu_q, slots, nt, "token_shift_multi")
    if mu.dim() != 2 or mu.shape[1] != d or out.shape != (mu.shape[0], nt, d) or state.dim() != 2 \
            or state.shape[1] != d:
        raise KernelError(f"token_shift_multi: h {tuple(h.shape)} out {tuple(out.shape)} mu {tuple(mu.shape)} "
                          f"state {tuple(state.shape)}")
    _check(library().ta_token_shift_multi(_stream(), c_int(_code(h.dtype)), _ptr(h), _ptr(out), _ptr(mu),
                                          c_int(mu.shape[0]), _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch),
                                          c_int(nt), c_int(d)))
    return out


def gemm_simple_batched(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[i] = a[i] @ w[i].T for 3-D views a [B, M, K], w [B, N, K], out [B, M, N] whose last
    axis is contiguous (any batch and row strides); float32 chains as ``gemm_simple``."""
    for t, n in ((a, "a"), (w, "w"), (out, "out")):
        _dev(t, n, contiguous=False)
        if t.dim() != 3 or t.stride(2) != 1:
            raise KernelError(f"gemm_simple_batched: {n} must be 3-D with a contiguous last axis")
    B, M, K = a.shape
    N = w.shape[1]
    if w.shape != (B, N, K) or out.shape != (B, M, N):
        raise KernelError(f"gemm_simple_batched: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if w.dtype != a.dtype and not (a.dtype == torch.bfloat16 and w.dtype == torch.float32):
        raise KernelError(f"gemm_simple_batched: activations are {a.dtype}, weights {w.dtype}")
    _check(library().ta_gemm_simple_batched(
        _stream(), c_int(_code(a.dtype)), c_int(_code(w.dtype)), c_int(_code(out.dtype)),
        _ptr(a), c_int(a.stride(1)), c_longlong(a.stride(0)), _ptr(w), c_int(w.stride(1)), c_longlong(w.stride(0)),
        _ptr(None), _ptr(out), c_int(out.stride(1)), c_longlong(out.stride(0)), c_int(M), c_int(N), c_int(K), c_int(B)))
    return out


# ------------------------------------------------------------------ the bonus recurrence ("wkv")
def wkv_recurrent(rkvg: torch.Tensor, low: torch.Tensor, heads: int, key_dim: int, value_dim: int, w2, w0, bonus,
                  state: torch.Tensor, cu_q, slots, o_out: torch.Tensor, decay: torch.Tensor) -> torch.Tensor:
    """Per head o_t = (S + diag(bonus) k_t v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T with
    w_t = exp(-exp(w2 @ tanh(low_t) + w0)) per key channel. rkvg [>= 3, nt, n] planes of r, k, v
    (n = H*dk = H*dv); low [nt, rank]; state [slots, H, dk, dv] float32; decay [nt, H*dk] float32
    scratch that receives the decays; o_out [gla_row_parts(dk), nt, H, dv] float32 planes."""
    _dev(rkvg, "rkvg"); _dev(low, "low", rkvg.dtype, contiguous=False)
    H, dk, dv = heads, key_dim, value_dim
    if rkvg.dim() != 3 or rkvg.shape[0] < 3 or dk != dv or rkvg.shape[2] != H * dk:
        raise KernelError(f"wkv_recurrent: planes {tuple(rkvg.shape)} for {H} heads of {dk} x {dv}")
    nt, n = rkvg.shape[1], rkvg.shape[2]
    nl, ls = _rows2d(low, "low")
    rank = low.shape[1]
    batch = _step_tables(cu_q, slots, nt, "wkv_recurrent")
    _dev(w2, "w2"); _dev(w0, "w0", torch.float32); _dev(bonus, "bonus", torch.float32)
    _dev(state, "state", torch.float32); _dev(o_out, "o_out", torch.float32); _dev(decay, "decay", torch.float32)
    if nl != nt or w2.shape != (n, rank) or w0.shape != (n,) or bonus.numel() != n or state.dim() != 4 \
            or state.shape[1:] != (H, dk, dv) or o_out.shape != (gla_row_parts(dk), nt, H, dv) \
            or decay.shape != (nt, n) or 3 * nt * n >= 2 ** 31:
        raise KernelError(f"wkv_recurrent: shapes do not fit {H} heads of {dk}: low {tuple(low.shape)} w2 "
                          f"{tuple(w2.shape)} state {tuple(state.shape)} o_out {tuple(o_out.shape)}")
    _check(library().ta_wkv_recurrent(
        _stream(), c_int(_code(rkvg.dtype)), c_int(_wcode(w2, rkvg.dtype, "wkv_recurrent")), _ptr(rkvg), c_int(n),
        c_int(0), c_int(nt * n), c_int(2 * nt * n), _ptr(low), c_int(ls), c_int(rank), _ptr(w2), _ptr(w0),
        _ptr(bonus), _ptr(decay), _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt), c_int(H),
        c_int(dk), c_int(dv), _ptr(o_out)))
    return o_out


_GATE_ACTS = {"silu": 0, "sigmoid": 1}


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, heads: int, value_dim: int,
                   weight: Optional[torch.Tensor], eps: float, out: torch.Tensor,
                   gate_act: str = "silu") -> torch.Tensor:
    """out = rms_norm(o per head) * weight * act(gate): o [parts, nt, H, dv] float32 planes that
    add up, gate [nt, H*dv] (contiguous rows), weight [dv] for all heads, [H*dv], or None (the
    plain division by the root mean square); act "silu" or "sigmoid". A norm over all heads at
    once is the call with heads = 1 and value_dim = the whole row."""
    _dev(o, "o", torch.float32); _dev(gate, "gate", contiguous=False); _dev(out, "out", gate.dtype)
    if weight is not None:
        _dev(weight, "weight", torch.float32)
    nt, gs = _rows2d(gate, "gate")
    H, dv = heads, value_dim
    if gate_act not in _GATE_ACTS:
        raise KernelError(f"head_norm_gate: unknown gate activation {gate_act!r}")
    if o.dim() != 4 or o.shape[1:] != (nt, H, dv) or out.shape != (nt, H * dv) or gate.shape[1] != H * dv \
            or (weight is not None and weight.numel() not in (dv, H * dv)):
        raise KernelError(f"head_norm_gate: o {tuple(o.shape)} gate {tuple(gate.shape)} out {tuple(out.shape)} "
                          f"weight {None if weight is None else tuple(weight.shape)}")
    wstride = dv if weight is not None and weight.numel() == H * dv and H > 1 else 0
    _check(library().ta_gla_out_act(_stream(), c_int(_code(gate.dtype)), _ptr(o), c_int(o.shape[0]), _ptr(gate),
                                    c_int(gs), c_longlong(0), _ptr(weight), c_int(wstride), c_float(eps),
                                    c_int(nt), c_int(H), c_int(dv), c_int(_GATE_ACTS[gate_act]), _ptr(out)))
    return out


def decay_recurrent(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, heads: int, key_dim: int,
                    value_dim: int, decays: torch.Tensor, q_scale: float, state: torch.Tensor, cu_q, slots,
                    o_out: torch.Tensor) -> torch.Tensor:
    """Linear attention with ONE fixed decay per head along every sequence: S <- decay_h S + k
    v^T, o = S^T (q_scale * q). q, k, v sit at columns q_off, k_off, v_off of the rows of
    ``proj`` (heads x key_dim, heads x key_dim, heads x value_dim). decays [H] float32 on the
    device; ``state`` [slots, H, dk, dv] float32; o_out [gla_row_parts(dk), nt, H, dv] float32
    planes that add up to the readout."""
    _dev(proj, "proj", contiguous=False)
    nt, stride = _rows2d(proj, "proj")
    H, dk, dv = heads, key_dim, value_dim
    batch = _step_tables(cu_q, slots, nt, "decay_recurrent")
    _dev(decays, "decays", torch.float32); _dev(state, "state", torch.float32); _dev(o_out, "o_out", torch.float32)
    ends = (q_off + H * dk, k_off + H * dk, v_off + H * dv)
    if min(q_off, k_off, v_off) < 0 or max(ends) > proj.shape[1] or decays.shape != (H,) or state.dim() != 4 \
            or state.shape[1:] != (H, dk, dv) or o_out.shape != (gla_row_parts(dk), nt, H, dv):
        raise KernelError(f"decay_recurrent: shapes do not fit {H} heads of {dk} / {dv}: proj {tuple(proj.shape)} "
                          f"offsets {(q_off, k_off, v_off)} decays {tuple(decays.shape)} state {tuple(state.shape)} "
                          f"o_out {tuple(o_out.shape)}")
    _check(library().ta_decay_recurrent(
        _stream(), c_int(_code(proj.dtype)), _ptr(proj), c_int(stride), c_int(q_off), c_int(k_off), c_int(v_off),
        _ptr(decays), c_float(q_scale), _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt), c_int(H),
        c_int(dk), c_int(dv), _ptr(o_out)))
    return o_out


def glu_limit(gate_up: torch.Tensor, out: torch.Tensor, limit: float, slope: float = 1.702,
              shift: float = 1.0) -> torch.Tensor:
    """Rows [gate | up] -> out = g * sigmoid(slope * g) * (u + shift) with g = min(gate, limit),
    u = clamp(up, -limit, limit); float32 inside. gate_up [nt, 2n], out [nt, n] contiguous."""
    _dev(gate_up, "gate_up", contiguous=False); _dev(out, "out", gate_up.dtype)
    nt, ld = _rows2d(gate_up, "gate_up")
    if gate_up.shape[1] % 2 or out.shape != (nt, gate_up.shape[1] // 2):
        raise KernelError(f"glu_limit: gate_up {tuple(gate_up.shape)} / out {tuple(out.shape)}")
    _check(library().ta_glu_limit(_stream(), c_int(_code(gate_up.dtype)), _ptr(gate_up), c_int(ld), _ptr(out),
                                  c_int(nt), c_int(out.shape[1]), c_float(limit), c_float(slope), c_float(shift)))
    return out


def normed_mean(deltas: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], eps: float,
                out: torch.Tensor) -> torch.Tensor:
    """out = mean over i of rms_norm(deltas[i], eps) * weights[i]: deltas float32 [nt, d] or
    [planes, nt, d] (planes added in order), weights float32 [d], out float32 [nt, d]."""
    _dev(out, "out", torch.float32)
    nt, d = out.shape
    n = len(deltas)
    if not 1 <= n <= 4 or len(weights) != n:
        raise KernelError(f"normed_mean: {n} branches with {len(weights)} weights (1 to 4 are taken)")
    planes, plane = [], []
    for i, (t, w) in enumerate(zip(deltas, weights)):
        _dev(t, f"deltas[{i}]", torch.float32); _dev(w, f"weights[{i}]", torch.float32)
        if t.dim() == 3 and t.shape[1:] == out.shape:
            planes.append(t.shape[0]); plane.append(nt * d)
        elif t.shape == out.shape:
            planes.append(1); plane.append(0)
        else:
            raise KernelError(f"normed_mean: deltas[{i}] is {tuple(t.shape)}, out {tuple(out.shape)}")
        if w.shape != (d,):
            raise KernelError(f"normed_mean: weights[{i}] is {tuple(w.shape)}, expected {(d,)}")
    dp = (c_void_p * n)(*[t.data_ptr() for t in deltas])
    wp = (c_void_p * n)(*[w.data_ptr() for w in weights])
    _check(library().ta_normed_mean(_stream(), c_int(n), dp, (c_int * n)(*planes), (c_longlong * n)(*plane), wp,
                                    c_float(eps), _ptr(out), c_int(nt), c_int(d)))
    return out


# ------------------------------------------------------------------ attention over one latent row per token
def latent_prepare(proj: torch.Tensor, q_rank: int, q_weight, cq, kv_offset: int, rank: int, rot: int,
                   rot_dims: int, k_weight, eps: float, angles, dest=None, kcache=None) -> None:
    """From rows ``proj`` [nt, >= ...]: cq [nt, q_rank] = rms_norm(first q_rank columns) *
    q_weight (q_rank 0: no query latent); with ``dest``: the cache row of every token takes
    rms_norm(columns kv_offset .. + rank) * k_weight and, behind it, the next ``rot`` columns
    with the first rot_dims of them rotated in pairs (2i, 2i + 1) by ``angles`` [nt, rot_dims/2, 2]."""
    _dev(proj, "proj", contiguous=False)
    nt, stride = _rows2d(proj, "proj")
    if q_rank:
        _dev(q_weight, "q_weight", torch.float32); _dev(cq, "cq", proj.dtype)
        if q_weight.shape != (q_rank,) or cq.shape != (nt, q_rank) or proj.shape[1] < q_rank:
            raise KernelError(f"latent_prepare: query latent of {q_rank}: weight {tuple(q_weight.shape)} cq {tuple(cq.shape)}")
    if dest is not None:
        _dev(dest, "dest", torch.int32); _dev(kcache, "kcache", proj.dtype); _dev(k_weight, "k_weight", torch.float32)
        if proj.shape[1] < kv_offset + rank + rot or k_weight.shape != (rank,) or dest.numel() != nt \
                or kcache.dim() != 4 or tuple(kcache.shape[1:3]) != (1, PAGE) or kcache.shape[3] < rank + rot:
            raise KernelError(f"latent_prepare: rows of {proj.shape[1]} / cache {tuple(kcache.shape)} do not fit a "
                              f"latent of {rank} + {rot} at column {kv_offset}")
        if rot_dims:
            _dev(angles, "angles", torch.float32)
            if tuple(angles.shape) != (nt, rot_dims // 2, 2):
                raise KernelError(f"latent_prepare: angles are {tuple(angles.shape)}, expected {(nt, rot_dims // 2, 2)}")
    _check(library().ta_latent_prepare(
        _stream(), c_int(_code(proj.dtype)), _ptr(proj), c_int(stride), c_int(q_rank), _ptr(q_weight if q_rank else None),
        _ptr(cq if q_rank else None), c_int(kv_offset), c_int(rank), c_int(rot), c_int(rot_dims),
        _ptr(k_weight if dest is not None else None), c_float(eps), _ptr(angles if rot_dims else None),
        _ptr(dest), _ptr(kcache if dest is not None else None),
        c_int(kcache.shape[3] if dest is not None else rank + rot), c_int(nt)))


def latent_query_rot(q: torch.Tensor, heads: int, nope: int, rot: int, rot_dims: int, angles, qa: torch.Tensor,
                     rank: int) -> torch.Tensor:
    """qa[t, h, rank:] = the last ``rot`` coordinates of head h of q[t], the first rot_dims of
    them rotated, then zeros up to the rows' width. q [nt, H*(nope + rot)], qa [nt, H, >= rank + rot]."""
    _dev(q, "q"); _dev(qa, "qa", q.dtype)
    nt = q.shape[0]
    if q.shape != (nt, heads * (nope + rot)) or qa.dim() != 3 or qa.shape[:2] != (nt, heads) or qa.shape[2] < rank + rot:
        raise KernelError(f"latent_query_rot: q {tuple(q.shape)} qa {tuple(qa.shape)}")
    if rot_dims:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (nt, rot_dims // 2, 2):
            raise KernelError(f"latent_query_rot: angles are {tuple(angles.shape)}")
    _check(library().ta_latent_query_rot(_stream(), c_int(_code(q.dtype)), _ptr(q), c_int(heads), c_int(nope),
                                         c_int(rot), c_int(rot_dims), _ptr(angles if rot_dims else None), _ptr(qa),
                                         c_int(rank), c_int(qa.shape[2]), c_int(nt)))
    return qa


LATENT_MAX_RANK = 512


def latent_row_width(rank: int, rot: int, dtype: torch.dtype) -> int:
    """Numbers a cached row (and a wide query) holds: rank + rot, rounded up to whole 16-byte
    pieces for bfloat16 so that the matrix-core kernel takes them (the rest is zero)."""
    return -(-(rank + rot) // 8) * 8 if dtype == torch.bfloat16 else rank + rot


def latent_key_shares(batch: int, max_qlen: int, heads: int, rank: int, width: int, max_kv_len: int,
                      window: Optional[int]) -> int:
    """Waves that share a row's keys in ``latent_attention`` on the matrix cores: one when the
    step's rows alone give the CUs enough work (then the kernel whose workgroups share their
    chunks runs), else enough to reach about two waves per SIMD while a share keeps at least
    two chunks of 32 keys. A function of the step's shape only."""
    rows = int(library().ta_latent_mfma_rows(c_int(rank), c_int(width), c_int(max_qlen), c_int(heads)))
    if rows == 0:
        return 1
    if max_qlen * heads >= 64 and batch * -(-max_qlen * heads // 64) >= 128:
        return 1        # enough workgroups of four tiles that share their chunks (the kernel for many rows)
    waves = batch * -(-max_qlen * heads // rows)
    keys = max_kv_len if not window else min(max_kv_len, window + max_qlen)
    chunks = keys // 32 + 2
    return max(1, min(chunks // 2, 2048 // max(waves, 1)))


def latent_attention(qa: torch.Tensor, out: torch.Tensor, kcache: torch.Tensor, block_table, cu_q, pos0,
                     max_qlen: int, rank: int, rot: int, scale: float, window=None, gate=None,
                     shares: int = 1) -> torch.Tensor:
    """Causal softmax attention of wide queries qa [nt, H, width] over cached rows kcache
    [pages, 1, PAGE, width] (width >= rank + rot, the rest zero); out [nt, H, rank] = weighted
    sums of the rows' first ``rank`` coordinates, times sigmoid(gate[t, h]) (gate [nt, >= H],
    contiguous rows). bfloat16 rows of whole 16-byte pieces run on the matrix cores, where
    ``shares`` waves divide a row's keys (``latent_key_shares``); all else on the vector ALU."""
    _dev(qa, "qa"); _dev(out, "out", qa.dtype); _dev(kcache, "kcache", qa.dtype)
    nt, H = qa.shape[0], qa.shape[1]
    width = qa.shape[2] if qa.dim() == 3 else -1
    if qa.dim() != 3 or width < rank + rot or out.shape != (nt, H, rank) or kcache.dim() != 4 \
            or tuple(kcache.shape[1:]) != (1, PAGE, width):
        raise KernelError(f"latent_attention: qa {tuple(qa.shape)} out {tuple(out.shape)} cache {tuple(kcache.shape)}")
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32); _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("latent_attention: cu_q / pos0 / block_table disagree about the batch size")
    gs = 0
    if gate is not None:
        _dev(gate, "gate", qa.dtype, contiguous=False)
        ng, gs = _rows2d(gate, "gate")
        if ng != nt or gate.shape[1] < H:
            raise KernelError(f"latent_attention: gate is {tuple(gate.shape)}")
    scratch = None
    if shares > 1:
        need = library().ta_latent_mfma_scratch
        need.restype = c_longlong
        floats = need(c_int(B), c_int(max_qlen), c_int(H), c_int(rank), c_int(width), c_int(shares))
        if floats > 0 and qa.dtype == torch.bfloat16:
            scratch = _scratch_floats(qa.device, floats)
        else:
            shares = 1
    _check(library().ta_latent_attention(
        _stream(), c_int(_code(qa.dtype)), _ptr(qa), _ptr(out), _ptr(kcache), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0), c_int(B), c_int(max_qlen), c_int(H), c_int(rank),
        c_int(rot), c_int(width), c_float(scale), c_int(window or 0), _ptr(gate), c_int(gs), c_int(shares),
        _ptr(scratch)))
    return out


# ------------------------------------------------------------------ routed feed-forward
_ROUTE_MODES = {"sigmoid": 0, "softmax": 1}
_MOE_ACTS = {None: 0, "gelu": 1, "gelu_tanh": 2, "relu2": 3, "silu": 4}


def moe_max_rows(pairs: int, experts: int) -> int:
    """Rows of the ordered pair list: every expert's run starts on a multiple of 16."""
    n = int(library().ta_moe_max_rows(c_int(pairs), c_int(experts)))
    if n < 0:
        raise KernelError(f"moe: {pairs} pairs of {experts} experts are too many rows")
    return n


def moe_route(logits: torch.Tensor, experts: int, top: int, chosen: torch.Tensor, weight: torch.Tensor,
              score: str = "sigmoid", renormalize: bool = False, bias: Optional[torch.Tensor] = None,
              groups: int = 1, keep_groups: int = 1):
    """chosen [nt, top] int32, weight [nt, top] float32: the ``top`` largest scores of the
    first ``experts`` columns of logits [nt, >= experts] float32 (lowest index among equals).
    bias [experts] float32: added to the logits first. "softmax" with ``renormalize`` is the
    softmax over the chosen logits alone. groups > 1: the experts form that many equal groups of
    neighbours, a group counts as its largest score, and only experts of the ``keep_groups`` best
    groups can be chosen."""
    _dev(logits, "logits", torch.float32, contiguous=False)
    nt, ld = _rows2d(logits, "logits")
    _dev(chosen, "chosen", torch.int32); _dev(weight, "weight", torch.float32)
    if score not in _ROUTE_MODES or logits.shape[1] < experts or chosen.shape != (nt, top) or weight.shape != (nt, top):
        raise KernelError(f"moe_route: logits {tuple(logits.shape)} chosen {tuple(chosen.shape)} score {score!r}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (experts,):
            raise KernelError(f"moe_route: bias is {tuple(bias.shape)}, expected {(experts,)}")
    if groups < 1 or experts % groups or not 1 <= keep_groups <= groups or top > keep_groups * (experts // groups):
        raise KernelError(f"moe_route: {experts} experts in {groups} groups of which {keep_groups} stay "
                          f"do not hold {top} choices")
    _check(library().ta_moe_route_groups(_stream(), _ptr(logits), _ptr(bias), c_int(ld), c_int(nt), c_int(experts),
                                         c_int(top), c_int(_ROUTE_MODES[score]), c_int(int(renormalize)),
                                         c_int(groups), c_int(keep_groups), _ptr(chosen), _ptr(weight)))
    return chosen, weight


def moe_plan(chosen: torch.Tensor, experts: int, row_pair: torch.Tensor, tile_expert: torch.Tensor,
             pair_row: torch.Tensor):
    """Orders the (token, choice) pairs by expert; see ``moe_max_rows`` for row_pair's size."""
    _dev(chosen, "chosen", torch.int32); _dev(row_pair, "row_pair", torch.int32)
    _dev(tile_expert, "tile_expert", torch.int32); _dev(pair_row, "pair_row", torch.int32)
    pairs = chosen.numel()
    rows = moe_max_rows(pairs, experts)
    if row_pair.numel() != rows or tile_expert.numel() != rows // 16 or pair_row.numel() != pairs:
        raise KernelError(f"moe_plan: {pairs} pairs of {experts} experts need {rows} rows")
    _check(library().ta_moe_plan(_stream(), _ptr(chosen), c_int(pairs), c_int(experts), c_int(rows), _ptr(row_pair),
                                 _ptr(tile_expert), _ptr(pair_row)))


def moe_gather(h: torch.Tensor, top: int, row_pair: torch.Tensor, weight, out: torch.Tensor) -> torch.Tensor:
    _dev(h, "h"); _dev(out, "out", h.dtype); _dev(row_pair, "row_pair", torch.int32)
    if weight is not None:
        _dev(weight, "weight", torch.float32)
    if out.shape != (row_pair.numel(), h.shape[1]):
        raise KernelError(f"moe_gather: out is {tuple(out.shape)}")
    _check(library().ta_moe_gather(_stream(), c_int(_code(h.dtype)), _ptr(h), c_int(h.shape[1]), c_int(top),
                                   _ptr(row_pair), _ptr(weight), _ptr(out), c_int(row_pair.numel())))
    return out


_MOE_FORMS = {"auto": 0, "split_k": 1, "direct": 2, "lds": 3}


def moe_gemm(a: torch.Tensor, w: torch.Tensor, tile_expert: torch.Tensor, out: torch.Tensor,
             act: Optional[str] = None, form: str = "auto") -> torch.Tensor:
    """out[rows of tile i] = act(a[rows] @ w[tile_expert[i]].T): a [rows, K], w [E, N, K], out
    [rows, N] in a's type or float32. form: which bfloat16 kernel runs ("auto": the shape
    decides between "lds", for many tiles, and "split_k", for few; "direct": operands straight
    from memory)."""
    if form not in _MOE_FORMS:
        raise KernelError(f"moe_gemm: unknown form {form!r}; known: {sorted(_MOE_FORMS)}")
    _dev(a, "a"); _dev(w, "w", a.dtype); _dev(out, "out"); _dev(tile_expert, "tile_expert", torch.int32)
    rows, K = a.shape
    if act not in _MOE_ACTS or w.dim() != 3 or w.shape[2] != K or out.shape != (rows, w.shape[1]) \
            or tile_expert.numel() * 16 != rows:
        raise KernelError(f"moe_gemm: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)} act {act!r}")
    _check(library().ta_moe_gemm_form(_stream(), c_int(_code(a.dtype)), c_int(_code(out.dtype)), _ptr(a), _ptr(w),
                                      _ptr(tile_expert), _ptr(out), c_int(rows), c_int(w.shape[1]), c_int(K),
                                      c_int(_MOE_ACTS[act]), c_int(_MOE_FORMS[form])))
    return out


def moe_combine(rows: torch.Tensor, top: int, pair_row: torch.Tensor, weight, shared, shared_gate,
                delta: torch.Tensor, extra: Optional[torch.Tensor] = None) -> torch.Tensor:
    """delta[t] = sum over the token's pairs of rows[pair_row] (* weight) + sigmoid(shared_gate[t,
    0]) * shared[t] (+ extra[t]); shared and extra [nt, d] or [planes, nt, d] float32;
    shared_gate float32 [nt, >= 1]. ``extra``: what another sublayer adds to the stream beside
    this one."""
    _dev(rows, "rows", torch.float32); _dev(pair_row, "pair_row", torch.int32); _dev(delta, "delta", torch.float32)
    nt, d = delta.shape
    if rows.shape[1] != d or pair_row.numel() != nt * top:
        raise KernelError(f"moe_combine: rows {tuple(rows.shape)} for {nt} tokens x {top}")
    planes, plane, gl = 1, 0, 0
    if weight is not None:
        _dev(weight, "weight", torch.float32)
    if shared is not None:
        _dev(shared, "shared", torch.float32)
        if shared.dim() == 3 and shared.shape[1:] == delta.shape:
            planes, plane = shared.shape[0], nt * d
        elif shared.shape != delta.shape:
            raise KernelError(f"moe_combine: shared is {tuple(shared.shape)}")
    if shared_gate is not None:
        _dev(shared_gate, "shared_gate", torch.float32, contiguous=False)
        ng, gl = _rows2d(shared_gate, "shared_gate")
        if ng != nt:
            raise KernelError(f"moe_combine: shared_gate is {tuple(shared_gate.shape)}")
    xplanes, xplane = 0, 0
    if extra is not None:
        _dev(extra, "extra", torch.float32)
        if extra.dim() == 3 and extra.shape[1:] == delta.shape:
            xplanes, xplane = extra.shape[0], nt * d
        elif extra.shape == delta.shape:
            xplanes = 1
        else:
            raise KernelError(f"moe_combine: extra is {tuple(extra.shape)}")
    _check(library().ta_moe_combine_extra(_stream(), _ptr(rows), c_int(d), c_int(top), _ptr(pair_row), _ptr(weight),
                                          _ptr(shared), c_int(planes), c_longlong(plane), _ptr(shared_gate),
                                          c_int(gl), _ptr(extra), c_int(xplanes), c_longlong(xplane), _ptr(delta),
                                          c_int(nt)))
    return delta


# ------------------------------------------------------------------ capped, sunk and gated softmax attention
_ROT_STYLES = {"half": 0, "interleaved": 1}


def qk_rotate_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                    own_kv: bool = True, bias: Optional[torch.Tensor] = None, angles: Optional[torch.Tensor] = None,
                    rot: int = 0, style: str = "interleaved", dest: Optional[torch.Tensor] = None,
                    kcache: Optional[torch.Tensor] = None, vcache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """On rows [q | k | v] of ``qkv`` (nh*dk, nkv*dk, nkv*dv columns; q alone without ``own_kv``):
    ``bias`` [columns] float32 is added, the first ``rot`` coordinates of every head of q and k turn by
    ``angles`` [nt, rot/2, 2] ("half": pairs (i, i + rot/2); "interleaved": (2i, 2i + 1)), q goes back
    in place, k and v are stored at ``dest`` into the cache layer. The cache's value rows may be wider
    than the values (vcache [pages, nkv, dvs, PAGE], dvs >= value_dim): the rest of a token's column is
    zeroed."""
    _dev(qkv, "qkv", contiguous=False)
    nt, stride = _rows2d(qkv, "qkv")
    own = num_kv_heads if own_kv else 0
    cols = num_heads * key_dim + own * (key_dim + value_dim)
    if qkv.shape[1] != cols:
        raise KernelError(f"qk_rotate_store: rows of {qkv.shape[1]}, expected {cols}")
    if style not in _ROT_STYLES or key_dim % 2 or rot % 2 or not 0 <= rot <= key_dim:
        raise KernelError(f"qk_rotate_store: {rot} rotated coordinates of heads of {key_dim}, pairing {style!r}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (cols,):
            raise KernelError(f"qk_rotate_store: bias is {tuple(bias.shape)}, expected {(cols,)}")
    if rot:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (nt, rot // 2, 2):
            raise KernelError(f"qk_rotate_store: angles are {tuple(angles.shape)}, expected {(nt, rot // 2, 2)}")
    else:
        angles = None
    if dest is not None:
        if not own_kv:
            raise KernelError("qk_rotate_store: a layer without keys and values of its own stores nothing")
        _dev(dest, "dest", torch.int32); _dev(kcache, "kcache", qkv.dtype); _dev(vcache, "vcache", qkv.dtype)
        store_dim = vcache.shape[2] if vcache.dim() == 4 else -1
        if store_dim < value_dim:
            raise KernelError(f"qk_rotate_store: cache value rows of {store_dim} cannot hold values of {value_dim}")
        _check_cache_layer("qk_rotate_store", kcache, vcache, num_kv_heads, key_dim, store_dim)
        if dest.numel() != nt:
            raise KernelError("qk_rotate_store: dest must hold one entry per token")
    _check(library().ta_qk_rotate_store(
        _stream(), c_int(_code(qkv.dtype)), _ptr(qkv), c_int(stride), _ptr(bias), _ptr(angles), c_int(rot),
        c_int(_ROT_STYLES[style]), _ptr(dest), _ptr(kcache if dest is not None else None),
        _ptr(vcache if dest is not None else None), c_int(nt), c_int(num_heads), c_int(num_kv_heads), c_int(own),
        c_int(key_dim), c_int(value_dim), c_int(store_dim if dest is not None else value_dim)))
    return qkv


def attention_sink(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads, num_kv_heads, key_dim,
                   value_dim, scale, window=None, softcap: Optional[float] = None, sink=None,
                   gate: Optional[torch.Tensor] = None, gate_dim: Optional[int] = None):
    """``attention_generic_dv`` with the options of a capped, sunk and gated softmax. softcap: score <-
    softcap * tanh(score / softcap) after the scale. sink: None; "unit": the denominator holds one more
    term exp(0) = 1; a float32 tensor [heads]: one more term exp(sink[head]). gate: rows [nt, >= heads *
    value_dim] of q's type whose sigmoid multiplies the result element by element. gate_dim: columns per
    head of the gate's rows where that is less than value_dim (a cache whose value rows are padded): the
    result's columns beyond it are not gated."""
    _dev(q, "q", contiguous=False); _dev(out, "out", q.dtype, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * key_dim or out.shape[1] != num_heads * value_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {key_dim} / {value_dim}")
    _dev(kcache, "kcache", q.dtype); _dev(vcache, "vcache", q.dtype)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, key_dim, value_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    gd = value_dim if gate_dim is None else int(gate_dim)
    if not 1 <= gd <= value_dim:
        raise KernelError(f"attention: gate columns per head {gd} outside [1, {value_dim}]")
    cap, mode, sink_t, gate, gs = _sink_args("attention", q, num_heads, gd, softcap, sink, gate)
    _check(library().ta_attention_generic_sink(
        _stream(), c_int(_code(q.dtype)), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache),
        _ptr(vcache), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0),
        c_int(B), c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(key_dim),
        c_int(value_dim), c_float(scale), c_int(window or 0), c_float(cap), c_int(mode),
        _ptr(sink_t), _ptr(gate), c_int(gs), c_int(gd)))
    return out


def _sink_args(what, q, num_heads, value_dim, softcap, sink, gate):
    """(softcap, sink mode, sink tensor, gate, gate stride) of the capped softmax's options, checked."""
    mode, sink_t = 0, None
    if isinstance(sink, str):
        if sink != "unit":
            raise KernelError(f"{what}: unknown sink {sink!r}")
        mode = 1
    elif sink is not None:
        _dev(sink, "sink", torch.float32)
        if sink.shape != (num_heads,):
            raise KernelError(f"{what}: sink is {tuple(sink.shape)}, expected {(num_heads,)}")
        mode, sink_t = 2, sink
    gs = 0
    if gate is not None:
        _dev(gate, "gate", q.dtype, contiguous=False)
        ng, gs = _rows2d(gate, "gate")
        if ng != q.shape[0] or gate.shape[1] < num_heads * value_dim:
            raise KernelError(f"{what}: gate rows are {tuple(gate.shape)}")
    if softcap is not None and not softcap > 0:
        raise KernelError(f"{what}: a cap must be positive, got {softcap}")
    return float(softcap or 0.0), mode, sink_t, gate, gs


def attention_rows_sink(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads, num_kv_heads,
                        head_dim, scale, window=None, softcap=None, sink=None, gate=None, gate_dim=None,
                        exact=True, through_lds=None):
    """``attention_rows`` (matrix cores, bfloat16, values as wide as the keys) with the options of
    ``attention_sink``. gate_dim: columns per head of the gate's rows (the values' own width where the
    cache pads them to the keys'); out's columns beyond it are not gated. exact: the softmax weights
    enter the second product as three bfloat16 pieces, so they keep 32 bits. through_lds 0 or 1 (None:
    1 from 256 rows on)."""
    if through_lds is None:
        through_lds = 1 if max_qlen * (num_heads // num_kv_heads) >= 256 and head_dim <= 192 else 0
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    gd = head_dim if gate_dim is None else int(gate_dim)
    cap, mode, sink_t, gate, gs = _sink_args("attention_rows_sink", q, num_heads, gd, softcap, sink, gate)
    _check(library().ta_attention_rows_sink_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache),
        _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0), c_int(B),
        c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_float(scale),
        c_int(window or 0), c_int(int(through_lds)), c_float(cap), c_int(int(exact)), c_int(mode), _ptr(sink_t),
        _ptr(gate), c_int(gs), c_int(gd)))
    return out


def attention_keys_sink(q, out, kcache, vcache, block_table, cu_q, pos0, max_kv_len, num_heads, num_kv_heads,
                        head_dim, scale, window=None, softcap=None, sink=None, gate=None, gate_dim=None,
                        exact=True, units=None, seq_units=None):
    """``attention_keys`` (single tokens on the matrix cores; q holds rotated heads, the cache the step's
    keys and values) with the options of ``attention_rows_sink``: the kernel whose four waves take a
    unit's pages in turn, and the merge, which adds the sink's share and applies the gate."""
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    if q.shape[0] != B:
        raise KernelError("attention_keys_sink: every sequence must bring exactly one token")
    if units is None:
        lens = [int(p) + 1 for p in pos0.tolist()]
        if max(lens) > block_table.shape[1] * PAGE:
            raise KernelError("attention_keys_sink: a sequence is longer than the block table")
        u, su = plan_key_units(lens, key_unit_count(B, num_kv_heads), tables=block_table.cpu().numpy())
        units = torch.from_numpy(u).to(q.device)
        seq_units = torch.from_numpy(su).to(q.device)
    _dev(units, "units", torch.int32); _dev(seq_units, "seq_units", torch.int32)
    if units.dim() != 2 or units.shape[1] != UNIT_INTS or tuple(seq_units.shape) != (B, 2) or units.shape[0] < B:
        raise KernelError(f"attention_keys_sink: units {tuple(units.shape)} / {tuple(seq_units.shape)} for {B} sequences")
    n_units = units.shape[0]
    gd = head_dim if gate_dim is None else int(gate_dim)
    cap, mode, sink_t, gate, gs = _sink_args("attention_keys_sink", q, num_heads, gd, softcap, sink, gate)
    need = library().ta_attention_keys_scratch
    need.restype = c_longlong
    scratch = _scratch_floats(q.device, need(c_int(n_units), c_int(num_heads), c_int(head_dim)))
    _check(library().ta_attention_keys_sink_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(pos0), c_int(B), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim),
        c_float(scale), c_int(window or 0), _ptr(units), _ptr(seq_units), c_int(n_units), c_int(4), _ptr(scratch),
        c_float(cap), c_int(int(exact)), c_int(mode), _ptr(sink_t), _ptr(gate), c_int(gs), c_int(gd)))
    return out


def keys_sink_fits(num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Whether ``attention_keys_sink`` takes this geometry: its four waves merge through 4 * (64 + rows *
    head size) floats of LDS, which have to fit 64 KB."""
    if head_dim % 32 or not 32 <= head_dim <= 256:
        return False
    group = num_heads // max(num_kv_heads, 1)
    return (4 * 64 + 4 * min(group, 32) * head_dim) * 4 <= 65536


# ------------------------------------------------------------------ short convolution, selective state space
_CONV_ACTS = {None: 0, "silu": 1}


def causal_conv(x: torch.Tensor, offset: int, channels: int, taps: torch.Tensor, out: torch.Tensor,
                conv_state: Optional[torch.Tensor], cu_q: torch.Tensor, slots: torch.Tensor, max_qlen: int,
                bias_in: Optional[torch.Tensor] = None, bias_out: Optional[torch.Tensor] = None,
                activation: Optional[str] = None, update: bool = True) -> torch.Tensor:
    """out[t, c] = act(bias_out[c] + sum_j taps[c, j] * u_(t - K + 1 + j)[c]) per sequence, u = columns
    [offset, offset + channels) of the rows of ``x`` plus ``bias_in``. Inputs before the step's first
    token of a sequence come from conv_state [slots, K - 1, channels] float32 (zero for a new sequence),
    which afterwards holds the sequence's last K - 1 inputs (``update``). taps [channels, K] float32;
    out [nt, channels] of x's type, not x itself. max_qlen: the most tokens a sequence brings (steps of
    single tokens take one kernel that also moves the memory on)."""
    _dev(x, "x", contiguous=False); _dev(out, "out", x.dtype, contiguous=False)
    nt, stride = _rows2d(x, "x")
    nto, ostride = _rows2d(out, "out")
    _dev(taps, "taps", torch.float32)
    if taps.dim() != 2 or taps.shape[0] != channels or nto != nt or out.shape[1] != channels or \
            offset < 0 or offset + channels > x.shape[1]:
        raise KernelError(f"causal_conv: x {tuple(x.shape)} columns {offset}..{offset + channels}, taps "
                          f"{tuple(taps.shape)}, out {tuple(out.shape)}")
    K = taps.shape[1]
    if activation not in _CONV_ACTS:
        raise KernelError(f"causal_conv: unknown activation {activation!r}")
    for name, b in (("bias_in", bias_in), ("bias_out", bias_out)):
        if b is not None:
            _dev(b, name, torch.float32)
            if b.shape != (channels,):
                raise KernelError(f"causal_conv: {name} is {tuple(b.shape)}, expected {(channels,)}")
    batch = _step_tables(cu_q, slots, nt, "causal_conv")
    if K > 1:
        _dev(conv_state, "conv_state", torch.float32)
        if conv_state.dim() != 3 or tuple(conv_state.shape[1:]) != (K - 1, channels):
            raise KernelError(f"causal_conv: state is {tuple(conv_state.shape)}, expected [slots, {K - 1}, {channels}]")
    if out.data_ptr() == x.data_ptr():
        raise KernelError("causal_conv: the result needs rows of its own")
    _check(library().ta_causal_conv(
        _stream(), c_int(_code(x.dtype)), _ptr(x), c_int(stride), c_int(offset), _ptr(bias_in), _ptr(taps),
        _ptr(bias_out), _ptr(conv_state if K > 1 else None), _ptr(cu_q), _ptr(slots), c_int(batch),
        c_int(nt), c_int(int(max_qlen)), c_int(channels), c_int(K), c_int(_CONV_ACTS[activation]), _ptr(out),
        c_int(ostride), c_int(int(update))))
    return out


def ssm_steps(proj: torch.Tensor, offset: int, heads: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
              dt: torch.Tensor, decay: torch.Tensor):
    """dt[t, h] = softplus(proj[t, offset + h] + dt_bias[h]) (no clamp), decay[t, h] = exp(-exp(a_log[h]) *
    dt[t, h]); both float32 [nt, heads]."""
    _dev(proj, "proj", contiguous=False)
    nt, stride = _rows2d(proj, "proj")
    _dev(dt_bias, "dt_bias", torch.float32); _dev(a_log, "a_log", torch.float32)
    _dev(dt, "dt", torch.float32); _dev(decay, "decay", torch.float32)
    if dt_bias.shape != (heads,) or a_log.shape != (heads,) or dt.shape != (nt, heads) or decay.shape != (nt, heads) \
            or offset < 0 or offset + heads > proj.shape[1]:
        raise KernelError(f"ssm_steps: proj {tuple(proj.shape)} columns {offset}..{offset + heads}, "
                          f"dt {tuple(dt.shape)}, decay {tuple(decay.shape)}")
    _check(library().ta_ssm_steps(_stream(), c_int(_code(proj.dtype)), _ptr(proj), c_int(stride), c_int(offset),
                                  _ptr(dt_bias), _ptr(a_log), c_int(nt), c_int(heads), _ptr(dt), _ptr(decay)))
    return dt, decay


def ssm_recurrent(xbc: torch.Tensor, x_off: int, b_off: int, c_off: int, heads: int, groups: int, state_dim: int,
                  head_dim: int, decay: torch.Tensor, dt: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
                  slots: torch.Tensor, o_out: torch.Tensor) -> torch.Tensor:
    """Per head h of group h // (heads / groups): S_t = decay[t, h] S_(t-1) + dt[t, h] B_t x_t^T (S is
    [state_dim, head_dim], float32, in ``state`` [slots, heads, state_dim, head_dim]), o_t = S_t^T C_t.
    x (heads * head_dim columns), B and C (groups * state_dim each) sit at column offsets of the rows of
    ``xbc``. o_out: [gla_row_parts(state_dim), nt, heads, head_dim] float32 planes that add up to o."""
    _dev(xbc, "xbc", contiguous=False)
    nt, stride = _rows2d(xbc, "xbc")
    if groups < 1 or heads % groups:
        raise KernelError(f"ssm_recurrent: {heads} heads do not divide into {groups} groups")
    for off, n in ((x_off, heads * head_dim), (b_off, groups * state_dim), (c_off, groups * state_dim)):
        if off < 0 or off + n > xbc.shape[1]:
            raise KernelError(f"ssm_recurrent: columns {off}..{off + n} of rows of {xbc.shape[1]}")
    _dev(decay, "decay", torch.float32); _dev(dt, "dt", torch.float32)
    _dev(state, "state", torch.float32); _dev(o_out, "o_out", torch.float32)
    if decay.shape != (nt, heads) or dt.shape != (nt, heads):
        raise KernelError(f"ssm_recurrent: decay {tuple(decay.shape)} / dt {tuple(dt.shape)}, expected {(nt, heads)}")
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, state_dim, head_dim):
        raise KernelError(f"ssm_recurrent: state is {tuple(state.shape)}")
    if tuple(o_out.shape) != (gla_row_parts(state_dim), nt, heads, head_dim):
        raise KernelError(f"ssm_recurrent: o_out is {tuple(o_out.shape)}")
    batch = _step_tables(cu_q, slots, nt, "ssm_recurrent")
    _check(library().ta_ssm_recurrent(
        _stream(), c_int(_code(xbc.dtype)), _ptr(xbc), c_int(stride), c_int(c_off), c_int(b_off), c_int(x_off),
        c_int(heads // groups), _ptr(decay), _ptr(dt), _ptr(state), _ptr(cu_q), _ptr(slots), c_int(batch), c_int(nt),
        c_int(heads), c_int(state_dim), c_int(head_dim), _ptr(o_out)))
    return o_out


def gated_group_norm(o: torch.Tensor, gate: torch.Tensor, gate_off: int, weight: Optional[torch.Tensor], eps: float,
                     groups: int, out: torch.Tensor, x: Optional[torch.Tensor] = None, x_off: int = 0,
                     skip: Optional[torch.Tensor] = None, head_dim: int = 0) -> torch.Tensor:
    """y = (sum of the planes of o + skip[head] * x) * silu(gate); the row is cut into ``groups`` equal
    parts, each divided by its own root mean square, times weight: the gate comes before the norm.
    o float32 [planes, nt, n]; gate at column gate_off of its rows, x at x_off of its rows (same type
    as out); skip float32 [n / head_dim]; out [nt, n]."""
    _dev(o, "o", torch.float32); _dev(out, "out")
    if o.dim() != 3 or out.dim() != 2 or tuple(o.shape[1:]) != tuple(out.shape):
        raise KernelError(f"gated_group_norm: o {tuple(o.shape)} / out {tuple(out.shape)}")
    parts, nt, n = o.shape
    if groups < 1 or n % groups:
        raise KernelError(f"gated_group_norm: rows of {n} do not divide into {groups} parts")
    _dev(gate, "gate", out.dtype, contiguous=False)
    ng, gs = _rows2d(gate, "gate")
    if ng != nt or gate_off < 0 or gate_off + n > gate.shape[1]:
        raise KernelError(f"gated_group_norm: gate rows {tuple(gate.shape)}, columns {gate_off}..{gate_off + n}")
    xs = 0
    if skip is not None:
        _dev(skip, "skip", torch.float32); _dev(x, "x", out.dtype, contiguous=False)
        nx, xs = _rows2d(x, "x")
        if head_dim < 1 or n % head_dim or skip.shape != (n // head_dim,) or nx != nt or x_off < 0 or x_off + n > x.shape[1]:
            raise KernelError(f"gated_group_norm: skip {tuple(skip.shape)} for heads of {head_dim} in rows of {n}")
    if weight is not None:
        _dev(weight, "weight", torch.float32)
        if weight.shape != (n,):
            raise KernelError(f"gated_group_norm: weight is {tuple(weight.shape)}, expected {(n,)}")
    _check(library().ta_gated_group_norm(
        _stream(), c_int(_code(out.dtype)), _ptr(o), c_int(parts), _ptr(x if skip is not None else None), c_int(xs),
        c_int(x_off), _ptr(skip), c_int(head_dim), _ptr(gate), c_int(gs), c_int(gate_off), _ptr(weight), c_float(eps),
        c_int(nt), c_int(n), c_int(groups), _ptr(out)))
    return out


def weighted_sum(deltas: Sequence[torch.Tensor], scales: Sequence[float], out: torch.Tensor) -> torch.Tensor:
    """out = sum over i of scales[i] * deltas[i]: deltas float32 [nt, d] or [planes, nt, d] (planes added
    in order), out float32 [nt, d]."""
    _dev(out, "out", torch.float32)
    nt, d = out.shape
    n = len(deltas)
    if not 1 <= n <= 4 or len(scales) != n:
        raise KernelError(f"weighted_sum: {n} branches with {len(scales)} scales (1 to 4 are taken)")
    planes, plane = [], []
    for i, t in enumerate(deltas):
        _dev(t, f"deltas[{i}]", torch.float32)
        if t.dim() == 3 and t.shape[1:] == out.shape:
            planes.append(t.shape[0]); plane.append(nt * d)
        elif t.shape == out.shape:
            planes.append(1); plane.append(0)
        else:
            raise KernelError(f"weighted_sum: deltas[{i}] is {tuple(t.shape)}, out {tuple(out.shape)}")
    dp = (c_void_p * n)(*[t.data_ptr() for t in deltas])
    _check(library().ta_weighted_sum(_stream(), c_int(n), dp, (c_int * n)(*planes), (c_longlong * n)(*plane),
                                     (c_float * n)(*[float(v) for v in scales]), _ptr(out), c_int(nt), c_int(d)))
    return out
