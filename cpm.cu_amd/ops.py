"""Python face of the HIP kernels: argument checks, then one launch each.

Tensors are torch tensors on the GPU, used as typed memory only; every function
launches on torch's current stream and allocates nothing.  Shapes are checked
here, on the host, before a pointer reaches a kernel; a size a kernel does not
take is refused with an error that names it.  There is no fallback: without a
GPU or without the built libraries these functions raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_ulonglong, c_void_p
from typing import Optional, Sequence, Tuple

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(t: torch.Tensor, name: str, dtype=None, shape: Optional[Sequence[Optional[int]]] = None):
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise KernelError(f"{name}: a GPU tensor is needed (no CPU path exists), got "
                          f"{getattr(t, 'device', type(t).__name__)}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous, strides {tuple(t.stride())} for shape {tuple(t.shape)}")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple('*' if s is None else s for s in shape)}")


def _p(t: Optional[torch.Tensor]):
    return c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


_fn_cache = {}


def _fn(module: str, name: str):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = _build.load(module)
        f = getattr(lib, name)
        f.restype = c_char_p
        _fn_cache[key] = f
    return f


def _check(msg):
    if msg:
        raise KernelError(msg.decode())


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float):
    """out[r] = float(table[ids[r]]) * scale;  table [V,H], ids int32 [n], out float32 [n,H]."""
    _need(table, "embed table", shape=(None, None))
    V, H = table.shape
    _need(ids, "embed ids", torch.int32, (None,))
    n = ids.shape[0]
    _need(out, "embed out", torch.float32, (n, H))
    _check(_fn("core", "cpmcu_embed")(_p(table), c_int(_code(table)), _p(ids), _p(out), c_int(n), c_int(H), c_int(V),
                                      c_float(scale), _stream()))


def add_rms_norm(x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float, weight: torch.Tensor,
                 eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None):
    """x += branch_scale * branch (in place; summed over the leading axis if branch is [P,n,H]);
    out = rmsnorm(x) * weight.  With ``rows`` (int32 [R]) only those rows are normed, into out [R,H],
    and x is left as it was."""
    _need(x, "norm x", torch.float32, (None, None))
    n, H = x.shape
    _need(weight, "norm weight", torch.float32, (H,))
    nparts, stride, bcode = 1, 0, F32
    if branch is not None:
        if branch.dim() == 3:
            _need(branch, "norm branch", shape=(None, n, H))
            nparts, stride = branch.shape[0], n * H
        else:
            _need(branch, "norm branch", shape=(n, H))
        bcode = _code(branch)
    if rows is not None:
        _need(rows, "norm rows", torch.int32, (None,))
        n_out = rows.shape[0]
    else:
        n_out = n
    _need(out, "norm out", shape=(n_out, H))
    _check(_fn("core", "cpmcu_add_rms_norm")(_p(x), _p(branch), c_int(bcode), c_int(nparts), c_long(stride),
                                             c_float(branch_scale), _p(weight), c_float(eps), _p(out),
                                             c_int(_code(out)), _p(rows), c_int(n_out), c_int(H), _stream()))


NORM_SLICE = 64        # columns a slice of add_norm_columns (common.h)

# The kernels of decode steps that own a strip of output columns over all of K (qkv_rope, proj_add_norm) and
# the norm cut by columns (add_norm_columns) save kernels of the chain, but every workgroup reads all of x.
# Up to 16 rows they win at every width measured (MI355X, 4,096 columns: norm 4.7 against 6.6 us at 8 rows).
# qkv_rope (workgroups spread evenly over the CUs) wins up to 32 rows (4,096 columns, q/k/v + rotary: 11.7
# against 18.2 us at 16 rows, 15.6 against 19.7 at 24, 16.5 against 21.3 at 32; it loses beyond: 24.6 against
# 21.3 at 48, 27.2 against 23.2 at 64), and proj_add_norm wins beyond 16 rows only while a workgroup's copy of
# x stays small (1,024 columns, 64 rows: 8.6 against 8.9 + 4.2 us).
STRIP_ROWS = 16
STRIP_MAX_ROWS = 64
STRIP_X_BYTES = 160 * 1024
QKV_ROPE_MAX_ROWS = 32


def strip_kernels_ok(n: int, K: int) -> bool:
    """Whether proj_add_norm (and the norm cut by columns) take a step of n rows of K columns."""
    return n <= STRIP_ROWS or (n <= STRIP_MAX_ROWS and n * K * 2 <= STRIP_X_BYTES)



class RowScale:
    """What a product needs to finish a norm cut by columns: the rows' sums of squares by slices of columns,
    float32 [n, slices] (a slice for every NORM_SLICE columns after add_norm_columns, for every 16 after
    proj_add_norm), and eps.  The product multiplies its rows by rsqrt(sum of the row's slices / H + eps), H
    being its own input width."""
    __slots__ = ("sums", "eps")

    def __init__(self, sums: torch.Tensor, eps: float):
        self.sums, self.eps = sums, float(eps)


def norm_slices(H: int) -> int:
    return -(-H // NORM_SLICE)


def add_norm_columns(x: torch.Tensor, branch: Optional[torch.Tensor], branch_scale: float, weight: torch.Tensor,
                     out: torch.Tensor, sums: torch.Tensor):
    """The norm of a step of few rows without its row factor: x += branch_scale * branch (in place; summed over
    the leading axis if branch is [P,n,H]); out = bfloat16(x * weight); sums[r, s] = sum of x[r]^2 over slice s.
    rmsnorm(x) * weight = out * rsqrt(sums.sum(1) / H + eps) row by row, which the product that reads `out`
    applies to its result (gemm_skinny, qkv_rope: row_scale)."""
    _need(x, "norm x", torch.float32, (None, None))
    n, H = x.shape
    if H % 4:
        raise KernelError(f"add_norm_columns: a width of {H} is no multiple of 4")
    _need(weight, "norm weight", torch.float32, (H,))
    nparts, stride, bcode = 1, 0, F32
    if branch is not None:
        if branch.dim() == 3:
            _need(branch, "norm branch", shape=(None, n, H))
            nparts, stride = branch.shape[0], n * H
        else:
            _need(branch, "norm branch", shape=(n, H))
        bcode = _code(branch)
    _need(out, "norm out", torch.bfloat16, (n, H))
    _need(sums, "norm row sums", torch.float32, (n, norm_slices(H)))
    _check(_fn("core", "cpmcu_add_norm_columns")(_p(x), _p(branch), c_int(bcode), c_int(nparts), c_long(stride),
                                                 c_float(branch_scale), _p(weight), _p(out), _p(sums), c_int(n),
                                                 c_int(H), _stream()))


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "clamped_swish": 2}


def gate_activation(activation):
    """(name, limit) of a gated pair's nonlinearity given as a name or as (name, limit).  'clamped_swish' is the one
    with a limit: g <- min(g, limit), up <- clamp(up, -limit, limit); the pair's product is g sigmoid(1.702 g) (up + 1)."""
    name, limit = activation if isinstance(activation, (tuple, list)) else (activation, 0.0)
    if name not in GATE_ACTIVATIONS:
        raise KernelError(f"gate nonlinearity '{name}' is not supported ({sorted(GATE_ACTIVATIONS)})")
    limit = float(limit or 0.0)
    if name == "clamped_swish" and not limit > 0:
        raise KernelError(f"gate nonlinearity 'clamped_swish' needs a positive limit, got {limit}")
    return name, limit


def _act(activation):
    """(c_int code, c_float limit) for the kernels."""
    name, limit = gate_activation(activation)
    return c_int(GATE_ACTIVATIONS[name]), c_float(limit)


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor, activation="silu"):
    """out[r,c] = act(gate_up[r,c]) * gate_up[r,c+I];  gate_up [n,2I], out [n,I]; act is SiLU or, with
    activation 'gelu_tanh', 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), or ('clamped_swish', limit)
    (gate_activation)."""
    _need(gate_up, "silu_mul input", shape=(None, None))
    n, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError(f"silu_mul: input width {two_i} is odd")
    _need(out, "silu_mul out", gate_up.dtype, (n, two_i // 2))
    _check(_fn("core", "cpmcu_silu_mul")(_p(gate_up), _p(out), c_int(_code(out)), c_int(n), c_int(two_i // 2),
                                         *_act(activation), _stream()))


def rope_store(qkv: torch.Tensor, q_out: torch.Tensor, nh: int, nkv: int, hd: int, positions: torch.Tensor,
               tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mscale: float,
               kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
               page_size: int, write_kv: bool = True):
    """Rotate q (and k), write q to q_out [n, nh*hd] and k, v into the paged cache.
    qkv [n, W] or float32 partial sums [P, n, W] with W >= (nh + 2 nkv) hd (nh*hd if not write_kv)."""
    if qkv.dim() == 3:
        _need(qkv, "rope qkv", torch.float32, (None, None, None))
        nparts, n, width = qkv.shape
        stride = n * width
    else:
        _need(qkv, "rope qkv", shape=(None, None))
        n, width = qkv.shape
        nparts, stride = 1, 0
    _need(q_out, "rope q_out", shape=(n, nh * hd))
    _need(positions, "rope positions", torch.int32, (n,))
    _need(tok_slot, "rope token slots", torch.int32, (n,))
    if inv_freq is not None:
        _need(inv_freq, "rope inv_freq", torch.float32, (hd // 2,))
    tw = 0
    if write_kv:
        _need(page_table, "rope page table", torch.int32, (None, None))
        tw = page_table.shape[1]
        _need(kpool, "rope key pool", q_out.dtype, (None, page_size, nkv * hd))
        _need(vpool, "rope value pool", q_out.dtype, tuple(kpool.shape))
    _check(_fn("core", "cpmcu_rope_store")(_p(qkv), c_long(width), c_int(_code(qkv)), c_int(nparts), c_long(stride),
                                           _p(q_out), c_int(_code(q_out)), c_int(n), c_int(nh), c_int(nkv), c_int(hd),
                                           _p(positions), _p(tok_slot), _p(inv_freq), c_float(mscale), _p(kpool),
                                           _p(vpool), _p(page_table), c_int(tw), c_int(page_size),
                                           c_int(1 if write_kv else 0), _stream()))


def gemm_nt_plain(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, alpha: float = 1.0):
    """out[m,N] = alpha * x[m,K] . w[N,K]^T with scalar float FMAs (any size, both element types)."""
    _need(x, "gemm x", shape=(None, None))
    M, K = x.shape
    _need(w, "gemm weight", x.dtype, (None, K))
    N = w.shape[0]
    _need(out, "gemm out", shape=(M, N))
    _check(_fn("gemm", "cpmcu_gemm_nt_plain")(_p(x), c_long(K), _p(w), c_long(K), _p(out), c_long(N), c_int(_code(x)),
                                              c_int(_code(out)), c_int(M), c_int(N), c_int(K), c_float(alpha),
                                              _stream()))


def attention_plain(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                    kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                    positions: torch.Tensor, tok_slot: torch.Tensor,
                    sel_blocks: Optional[torch.Tensor] = None, sel_count: Optional[torch.Tensor] = None,
                    block_size: int = 0, head_slopes: Optional[torch.Tensor] = None):
    """Causal GQA attention of n query tokens over their sequences' cached keys (plain kernel).  head_slopes
    (float32 [nh]): the score of key j for the query at position p is lowered by head_slopes[h] * (p - j)."""
    _need(q, "attention q", shape=(None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", q.dtype, (n, nh * hd))
    _need(kpool, "attention key pool", q.dtype, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", q.dtype, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    max_sel = 0
    if sel_count is not None:
        _need(sel_count, "attention block counts", torch.int32, (n, nkv))
        _need(sel_blocks, "attention block list", torch.int32, (n, nkv, None))
        max_sel = sel_blocks.shape[2]
    if head_slopes is not None:
        _need(head_slopes, "attention head slopes", torch.float32, (nh,))
    _check(_fn("attention", "cpmcu_attention_plain")(
        _p(q), _p(out), c_int(_code(q)), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale), _p(kpool),
        _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot),
        _p(sel_blocks), _p(sel_count), c_int(max_sel), c_int(block_size), _p(head_slopes), _stream()))


MFMA_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128)


def attention_mfma_ok(q: torch.Tensor, hd: int, page_size: int, block_size: int = 0) -> bool:
    return (q.dtype == torch.bfloat16 and hd in MFMA_HEAD_DIMS and page_size % 32 == 0
            and (block_size == 0 or block_size % 32 == 0))


def attention_mfma(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                   kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                   positions: torch.Tensor, tok_slot: torch.Tensor, n_splits: int = 1,
                   part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                   sel_blocks: Optional[torch.Tensor] = None, sel_count: Optional[torch.Tensor] = None,
                   block_size: int = 0, waves_per_group: int = 0, last_blocks_first: int = 0):
    """bf16 attention on the matrix cores (head_dim 16, 32, ... 128; pages and key blocks multiples of 32).
    With n_splits > 1 every token's keys are shared among n_splits wavefronts and merged afterwards;
    part_o float32 [n, nh, n_splits, hd] and part_ml float32 [n, nh, n_splits, 2] are its scratch.
    last_blocks_first: that many blocks at the end of every block list (the window that neighbouring tokens
    share) are visited before the others; it changes the order of the sums only."""
    _need(q, "attention q", torch.bfloat16, (None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", torch.bfloat16, (n, nh * hd))
    _need(kpool, "attention key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    max_sel = 0
    if sel_count is not None:
        _need(sel_count, "attention block counts", torch.int32, (n, nkv))
        _need(sel_blocks, "attention block list", torch.int32, (n, nkv, None))
        max_sel = sel_blocks.shape[2]
    if n_splits > 1:
        _need(part_o, "attention partial outputs", torch.float32, (n, nh, n_splits, hd))
        _need(part_ml, "attention partial max/sum", torch.float32, (n, nh, n_splits, 2))
    _check(_fn("attention", "cpmcu_attention_mfma")(
        _p(q), _p(out), _p(part_o), _p(part_ml), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale),
        _p(kpool), _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions),
        _p(tok_slot), _p(sel_blocks), _p(sel_count), c_int(max_sel), c_int(block_size), c_int(n_splits),
        c_int(waves_per_group), c_int(last_blocks_first), _stream()))


def attention_prefill_tokens_per_wave(nh: int, nkv: int, tiles_per_wave: int = 4) -> int:
    lib = _build.load("attention")
    lib.cpmcu_attention_prefill_tokens_per_wave.restype = c_int
    return int(lib.cpmcu_attention_prefill_tokens_per_wave(c_int(nh), c_int(nkv), c_int(tiles_per_wave)))


def attention_prefill_shape(n_tokens: int, nh: int, nkv: int, hd: int):
    """(tiles a wavefront, wavefronts a workgroup) for the prompt kernel.  Measured on the MI355X at head size
    128, 32 heads in 2 groups, one prompt of 512 / 2,048 / 8,192 / 32,768 tokens, in us:
      2 tiles, 1 / 2 / 4 wavefronts:  25 / 20 / 19    95 / 75 / 90    894 / 819 / 835   11.3 / 11.6 / 11.8 ms
      4 tiles, 1 / 2 / 4 wavefronts:  37 / 26 / 24   123 / 86 / 116   888 / 904 / 1058  13.7 / 13.4 / 14.1 ms
    Two tiles of 16 rows a wavefront leave room for two wavefronts a SIMD; wavefronts that share a group of
    tiles take the chunks of keys in turn, which evens out the causal triangle of short prompts."""
    if n_tokens <= 1024:
        return 2, 4
    return 2, (2 if n_tokens < 16384 else 1)


def attention_prefill_mfma(q: torch.Tensor, out: torch.Tensor, tiles: torch.Tensor, nh: int, nkv: int, hd: int,
                           scale: float, kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor,
                           page_size: int, positions: torch.Tensor, tok_slot: torch.Tensor, tiles_per_wave: int = 4,
                           waves_per_group: int = 1):
    """Dense causal bf16 attention for prompts: tiles int32 [T, 2] = (first packed token, tokens), each a run of
    consecutive tokens of one sequence, at most attention_prefill_tokens_per_wave(nh, nkv, tiles_per_wave) long."""
    _need(q, "attention q", torch.bfloat16, (None, nh * hd))
    n = q.shape[0]
    _need(out, "attention out", torch.bfloat16, (n, nh * hd))
    _need(tiles, "attention tiles", torch.int32, (None, 2))
    _need(kpool, "attention key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "attention value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    _check(_fn("attention", "cpmcu_attention_prefill_mfma")(
        _p(q), _p(out), c_int(tiles.shape[0]), _p(tiles), c_int(tiles_per_wave), c_int(waves_per_group), c_int(nh),
        c_int(nkv), c_int(hd),
        c_float(scale),
        _p(kpool), _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions),
        _p(tok_slot), _stream()))


def prefill_tiles(q_lens: Sequence[int], tokens_per_wave: int, device) -> torch.Tensor:
    """Runs of at most tokens_per_wave consecutive tokens of one sequence, covering the packed batch."""
    tiles = []
    start = 0
    for q in q_lens:
        for a in range(0, q, tokens_per_wave):
            tiles.append((start + a, min(tokens_per_wave, q - a)))
        start += q
    return torch.tensor(tiles, dtype=torch.int32).to(device)


_cu_count = None


def compute_units() -> int:
    """CUs of the current GPU (256 on the MI355X, which is also what the heuristics below were measured on and
    what they assume when no GPU is visible)."""
    global _cu_count
    if _cu_count is None:
        _cu_count = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                     if torch.cuda.is_available() else 256)
    return _cu_count


def attention_splits(n_tokens: int, nkv: int, group: int, max_keys: int) -> int:
    """Shares of a token's keys for steps of few tokens.  Measured on the MI355X (head size 128, 2 kv heads,
    workgroups of 4 wavefronts, graph replay over keys that come from memory, attention + merge, in us for
    1/2/4/8/16/32 shares):
      8 sequences at 4,096 keys 38/24/17/13/12.5/14, at 16,384 keys 146/80/47/32/30/30, at 32,768 279/150/87/59/53/55;
      16 sequences at 4,096 keys 43/30/21/18/20/23; 24 sequences 44/34/24/27/27/31; 32 sequences 48/32/30/32/34/39;
      64 sequences 55/52/53/57/59/71;
      one sequence at 4,096 keys 22/15/11/8.8/7.9/7.6, at 16,384 keys 140/74/41/25/17/12.5, at 65,536 531/275/140/76/46/28;
      4 sequences at 32,768 keys 278/148/80/49/32/30.
    So: as many shares as give about 256 workgroups in all, one for every CU (a CU takes in ~30 GB/s however
    much it has in flight; the merge kernel costs ~3 us whatever the number of shares up to 32), a share of at
    least 128 keys, at most 32 shares (beyond 32 the merge kernel no longer holds every share's output in
    registers: one sequence at 32,000 keys, whole step, 3.89 ms with 64 shares against 3.60 with 32).  A step
    that has 128 workgroups or more by itself takes two shares from 4,096 keys on (they even out the
    workgroups' ends) and one below (no merge kernel: 64 sequences of the 0.5B shape)."""
    cus = compute_units()
    if n_tokens > cus:
        return 1
    groups = n_tokens * nkv * -(-group // 16)
    want = max(1, cus // max(groups, 1))
    if groups >= cus // 2:
        want = 2 if max_keys >= 4096 else 1
    return max(1, min(want, max_keys // 128, 32))


def compress_keys(kpool: torch.Tensor, ckpool: torch.Tensor, nkv: int, page_table: torch.Tensor, page_size: int,
                  positions: torch.Tensor, tok_slot: torch.Tensor, kernel_size: int, kernel_stride: int):
    """Write the compressed keys (means of kernel_size keys, every kernel_stride) that the step's tokens complete.
    The keys lie in their pages as rope_store writes them; a compressed key is a plain row [kv head][d]."""
    _need(kpool, "compress key pool", shape=(None, page_size, None))
    width = kpool.shape[2]
    if nkv <= 0 or width % nkv:
        raise KernelError(f"compress_keys: rows of {width} elements do not hold {nkv} kv heads")
    if kernel_stride <= 0 or page_size % kernel_stride:
        raise KernelError(f"compress_keys: kernel_stride {kernel_stride} must divide the cache page of {page_size} tokens")
    _need(ckpool, "compressed key pool", kpool.dtype, (kpool.shape[0], page_size // kernel_stride, width))
    _need(page_table, "compress page table", torch.int32, (None, None))
    _need(positions, "compress positions", torch.int32, (None,))
    n = positions.shape[0]
    _need(tok_slot, "compress token slots", torch.int32, (n,))
    _check(_fn("sparse", "cpmcu_compress_keys")(_p(kpool), _p(ckpool), c_int(_code(kpool)), c_int(n), c_int(nkv),
                                                c_int(width // nkv), _p(page_table), c_int(page_table.shape[1]), c_int(page_size),
                                                _p(positions), _p(tok_slot), c_int(kernel_size), c_int(kernel_stride),
                                                _stream()))


def sparse_select_scratch(dtype: torch.dtype, n: int, nh: int, nkv: int, hd: int, max_pos: int, kernel_size: int,
                          kernel_stride: int, block_size: int, force_plain=False) -> int:
    """Floats of scratch that sparse_select wants for a step of n tokens at positions up to max_pos (0: none).
    bf16 steps of few tokens run as three kernels of many small workgroups through it; contexts whose scores
    and ranking arrays exceed a workgroup's LDS keep them there instead (any step, both element types)."""
    lib = _build.load("sparse")
    f = lib.cpmcu_sparse_select_scratch
    f.restype = c_long
    return int(f(c_int(_DT[dtype]), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_int(kernel_size), c_int(kernel_stride),
                 c_int(block_size), c_int(max_pos), c_int(int(force_plain))))


def sparse_select(q: torch.Tensor, ckpool: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                  page_table: torch.Tensor, page_size: int, positions: torch.Tensor, tok_slot: torch.Tensor,
                  kernel_size: int, kernel_stride: int, block_size: int, init_blocks: int, topk: int,
                  window_blocks: int, dense_len: int, max_pos: int, sel_blocks: torch.Tensor, sel_count: torch.Tensor,
                  force_plain=False, scratch: Optional[torch.Tensor] = None):
    """Block list per (token, kv head): sel_count -1 = dense, else the ascending blocks to attend to.
    scratch: float32 of at least sparse_select_scratch(...) elements, if that is not 0.
    force_plain: True = the plain kernel; 2 = steps of few tokens with the normalising kernel kept apart, as for
    contexts too long for the fused form (for tests)."""
    _need(q, "select q", shape=(None, nh * hd))
    n = q.shape[0]
    _need(ckpool, "select compressed keys", q.dtype, (None, page_size // max(kernel_stride, 1), nkv * hd))
    _need(page_table, "select page table", torch.int32, (None, None))
    _need(positions, "select positions", torch.int32, (n,))
    _need(tok_slot, "select token slots", torch.int32, (n,))
    _need(sel_count, "select counts", torch.int32, (n, nkv))
    _need(sel_blocks, "select block list", torch.int32, (n, nkv, None))
    if scratch is not None:
        _need(scratch, "select scratch", torch.float32, (None,))
    _check(_fn("sparse", "cpmcu_sparse_select")(
        _p(q), _p(ckpool), c_int(_code(q)), c_int(n), c_int(nh), c_int(nkv), c_int(hd), c_float(scale),
        _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot),
        c_int(kernel_size), c_int(kernel_stride), c_int(block_size), c_int(init_blocks), c_int(topk),
        c_int(window_blocks), c_int(dense_len), c_int(max_pos), _p(sel_blocks), _p(sel_count),
        c_int(sel_blocks.shape[2]), c_int(int(force_plain)), _p(scratch),
        c_long(scratch.numel() if scratch is not None else 0), _stream()))


def _ld(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous (a slice of columns of a wider tensor is)."""
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise KernelError(f"{name}: a GPU tensor is needed (no CPU path exists)")
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name}: rows must be contiguous, strides {tuple(t.stride())} for shape {tuple(t.shape)}")
    return int(t.stride(0)) if t.shape[0] > 1 else max(int(t.stride(0)), int(t.shape[1]))


def rms_norm_groups(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out: torch.Tensor, groups: int = 1,
                    gate: Optional[torch.Tensor] = None, gate_after=False,
                    divisor: Optional[torch.Tensor] = None):
    """out[r] = v / sqrt(mean(v^2) + eps) * weight, group by group (``groups`` equal parts of a row, each by its
    own root mean square), v = x * silu(gate) when a gate is given (the gate comes before the norm); with
    ``gate_after`` v = x and the result is multiplied by sigmoid(gate) instead (by silu(gate) with gate_after="silu").  ``divisor`` (float32 [n, groups]):
    a group's values are divided by its number first.  x, gate and out may be column slices of wider tensors;
    statistics in float."""
    ldx, ldo = _ld(x, "norm x"), _ld(out, "norm out")
    n, width = x.shape
    if groups <= 0 or width % groups:
        raise KernelError(f"rms_norm_groups: {width} columns do not split into {groups} equal groups")
    if tuple(out.shape) != (n, width):
        raise KernelError(f"norm out: shape {tuple(out.shape)}, expected {(n, width)}")
    if weight is not None:
        _need(weight, "norm weight", torch.float32, (width,))
    ldz = 0
    if gate is not None:
        ldz = _ld(gate, "norm gate")
        if tuple(gate.shape) != (n, width):
            raise KernelError(f"norm gate: shape {tuple(gate.shape)}, expected {(n, width)}")
    if divisor is not None:
        _need(divisor, "norm divisor", torch.float32, (n, groups))
    _check(_fn("norms", "cpmcu_rms_norm_groups")(_p(x), c_long(ldx), c_int(_code(x)), _p(gate), c_long(ldz),
                                                 c_int(_code(gate) if gate is not None else 0), _p(weight), _p(out),
                                                 c_long(ldo), c_int(_code(out)), c_int(n), c_int(groups),
                                                 c_int(width // groups), c_float(eps), c_int(2 if gate_after == "silu" else (1 if gate_after else 0)),
                                                 _p(divisor), _stream()))


def branch_norm_add_norm(x: torch.Tensor, branch: torch.Tensor, branch_weight: torch.Tensor, branch_eps: float,
                         weight: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
                         rows: Optional[torch.Tensor] = None):
    """x += rmsnorm(branch) * branch_weight (in place; the branch summed over its leading axis first if it is
    [P,n,H]); out = rmsnorm(x) * weight.  With ``rows`` (int32 [R]) only those rows are computed, into out
    [R,H], and x is left as it was.  out None: only the residual is updated."""
    _need(x, "norm x", torch.float32, (None, None))
    n, H = x.shape
    nparts, stride = 1, 0
    if branch.dim() == 3:
        _need(branch, "norm branch", shape=(None, n, H))
        nparts, stride = branch.shape[0], n * H
    else:
        _need(branch, "norm branch", shape=(n, H))
    _need(branch_weight, "branch norm weight", torch.float32, (H,))
    n_out = n
    if rows is not None:
        _need(rows, "norm rows", torch.int32, (None,))
        n_out = rows.shape[0]
    if out is not None:
        _need(weight, "norm weight", torch.float32, (H,))
        _need(out, "norm out", shape=(n_out, H))
    _check(_fn("norms", "cpmcu_branch_norm_add_norm")(_p(x), _p(branch), c_int(_code(branch)), c_int(nparts),
                                                      c_long(stride), _p(branch_weight), c_float(branch_eps),
                                                      _p(weight), c_float(eps), _p(out),
                                                      c_int(_code(out) if out is not None else 0), _p(rows),
                                                      c_int(n_out), c_int(H), _stream()))


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float, out: torch.Tensor):
    """out = a z/rms(z) + b z^2/rms(z^2) + c z^3/rms(z^3) + e row by row, (a, b, c, e) = coef (float32 [4] on the
    device), powers element by element, rms(v) = sqrt(mean(v^2) + eps); z [n,F] or float partial sums [P,n,F]."""
    nparts, stride = 1, 0
    if z.dim() == 3:
        _need(z, "poly_norm z", torch.float32, (None, None, None))
        nparts, n, F = z.shape
        stride = n * F
    else:
        _need(z, "poly_norm z", shape=(None, None))
        n, F = z.shape
    _need(coef, "poly_norm coefficients", torch.float32, (4,))
    _need(out, "poly_norm out", shape=(n, F))
    _check(_fn("norms", "cpmcu_poly_norm")(_p(z), c_int(_code(z)), c_int(nparts), c_long(stride), _p(coef), _p(out),
                                           c_int(_code(out)), c_int(n), c_int(F), c_float(eps), _stream()))


def conv_silu(u: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
              out: torch.Tensor, cu_q: torch.Tensor, seq_slot: torch.Tensor, max_q: int, update_state: bool = True,
              in_bias: Optional[torch.Tensor] = None, activation: bool = True):
    """Causal convolution per channel over each sequence's tokens, then SiLU.  u [n,C] (may be a column slice),
    weight float32 [C,taps] (last column = the current token's), state float32 [slots, taps-1, C] = each slot's
    last inputs (zeros before a sequence's start), out float32 [n,C].  cu_q int32 [B+1], seq_slot int32 [B];
    max_q: the longest run of tokens a sequence brings.  The state moves on to the step's last inputs.
    in_bias (float32 [C]): the inputs are u + in_bias (a projection's bias not yet added; the state holds them
    with it).  Without ``activation`` the convolution's result is written as it is."""
    ldu = _ld(u, "conv input")
    n, C = u.shape
    _need(weight, "conv weight", torch.float32, (C, None))
    taps = weight.shape[1]
    if bias is not None:
        _need(bias, "conv bias", torch.float32, (C,))
    if in_bias is not None:
        _need(in_bias, "conv input bias", torch.float32, (C,))
    if taps > 1:
        _need(state, "conv state", torch.float32, (None, taps - 1, C))
    _need(out, "conv out", torch.float32, (n, C))
    _need(cu_q, "conv sequence starts", torch.int32, (None,))
    B = cu_q.shape[0] - 1
    _need(seq_slot, "conv sequence slots", torch.int32, (B,))
    _check(_fn("ssm", "cpmcu_conv_silu")(_p(u), c_long(ldu), c_int(_code(u)), _p(weight), _p(bias), _p(state), _p(out),
                                         _p(cu_q), _p(seq_slot), c_int(B), c_int(max_q), c_int(C), c_int(taps),
                                         c_int(1 if update_state else 0), _p(in_bias),
                                         c_int(0 if activation else 1), _stream()))


def ssm_scan(xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
             state: torch.Tensor, y: torch.Tensor, cu_q: torch.Tensor, seq_slot: torch.Tensor, heads: int, P: int,
             N: int, groups: int, write_state: bool = True):
    """The state-space recurrence over each sequence's tokens, in float: per head h (group h // (heads/groups)),
    d = softplus(dt + dt_bias[h]); S <- exp(-exp(A_log[h]) d) S + d B x^T; y = S^T C + D[h] x.
    xbc float32 [n, heads*P + 2*groups*N] = [x | B | C]; dt [n, heads] (may be a column slice);
    state float32 [slots, heads, P, N]; y float32 [n, heads*P]."""
    _need(xbc, "scan inputs", torch.float32, (None, heads * P + 2 * groups * N))
    n = xbc.shape[0]
    lddt = _ld(dt, "scan step sizes")
    if tuple(dt.shape) != (n, heads):
        raise KernelError(f"scan step sizes: shape {tuple(dt.shape)}, expected {(n, heads)}")
    for t, name in ((dt_bias, "dt_bias"), (A_log, "A_log"), (D, "D")):
        _need(t, f"scan {name}", torch.float32, (heads,))
    _need(state, "scan state", torch.float32, (None, heads, P, N))
    _need(y, "scan out", torch.float32, (n, heads * P))
    _need(cu_q, "scan sequence starts", torch.int32, (None,))
    B = cu_q.shape[0] - 1
    _need(seq_slot, "scan sequence slots", torch.int32, (B,))
    _check(_fn("ssm", "cpmcu_ssm_scan")(_p(xbc), c_long(xbc.shape[1]), _p(dt), c_long(lddt), c_int(_code(dt)),
                                        _p(dt_bias), _p(A_log), _p(D), _p(state), _p(y), _p(cu_q), _p(seq_slot),
                                        c_int(B), c_int(heads), c_int(P), c_int(N), c_int(groups),
                                        c_int(1 if write_state else 0), _stream()))


ROTATE_TO_ROWS, ROTATE_TO_KEYS, ROTATE_TO_VALUES = 0, 1, 2


def rotate_copy(src: torch.Tensor, src_off: int, src_head_stride: int, heads: int, width: int, rot_dims: int,
                positions: torch.Tensor, inv_freq: Optional[torch.Tensor], mag: float, dst: torch.Tensor,
                mode: int = ROTATE_TO_ROWS, dst_off: int = 0, dst_head_stride: int = 0,
                tok_slot: Optional[torch.Tensor] = None, page_table: Optional[torch.Tensor] = None,
                page_size: int = 0, pool_heads: int = 0, pool_hd: int = 0):
    """For every (token, head): copy ``width`` features from src[t, src_off + h*src_head_stride ...], the first
    ``rot_dims`` of them rotated by position (feature i pairs with i + rot_dims/2; angle = position *
    inv_freq[i]; cos and sin times ``mag``), to rows of ``dst`` (ROTATE_TO_ROWS: dst[t, dst_off +
    h*dst_head_stride ...]) or into the paged cache in the key or value layout, at feature dst_off of cached
    head h (``pool_heads`` heads of ``pool_hd`` features a token)."""
    ld_src = _ld(src, "rotate source")
    n = src.shape[0]
    if src_off < 0 or src_off + (heads - 1) * src_head_stride + width > src.shape[1]:
        raise KernelError(f"rotate_copy: {heads} heads of {width} features from column {src_off} (stride "
                          f"{src_head_stride}) do not fit rows of {src.shape[1]}")
    _need(positions, "rotate positions", torch.int32, (n,))
    if rot_dims:
        _need(inv_freq, "rotate inv_freq", torch.float32, (rot_dims // 2,))
    ld_dst, tw = 0, 0
    if mode == ROTATE_TO_ROWS:
        ld_dst = _ld(dst, "rotate destination")
        if dst.shape[0] != n or dst_off < 0 or dst_off + (heads - 1) * dst_head_stride + width > dst.shape[1]:
            raise KernelError(f"rotate_copy: {heads} heads of {width} features to column {dst_off} (stride "
                              f"{dst_head_stride}) do not fit {tuple(dst.shape)}")
    else:
        _need(tok_slot, "rotate token slots", torch.int32, (n,))
        _need(page_table, "rotate page table", torch.int32, (None, None))
        _need(dst, "rotate pool", shape=(None, page_size, pool_heads * pool_hd))
        tw = page_table.shape[1]
    _check(_fn("attention_general", "cpmcu_rotate_copy")(
        _p(src), c_int(_code(src)), c_long(ld_src), c_long(src_head_stride), c_long(src_off), _p(dst),
        c_int(_code(dst)), c_int(mode), c_long(ld_dst), c_long(dst_head_stride), c_long(dst_off), c_int(n),
        c_int(heads), c_int(width), c_int(rot_dims), _p(positions), _p(tok_slot), _p(inv_freq), c_float(mag),
        _p(page_table), c_int(tw), c_int(page_size), c_int(pool_heads), c_int(pool_hd), _stream()))


def qkv_rotate_store(qkv: torch.Tensor, q_out: torch.Tensor, nh: int, nkv: int, dk: int, dv: int, rot_dims: int,
                     positions: torch.Tensor, tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mag: float,
                     kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
                     page_size: int, write_kv: bool = True, interleaved: bool = False):
    """rotate_copy three times in one launch: a row of qkv is [q: nh*dk | k: nkv*dk | v: nkv*dv]; q goes, rotated
    in its first rot_dims features, to q_out [n, nh*dk], k rotated into the key pages, v into the value pages
    (pools whose heads may be padded to a multiple of 16 features).  ``interleaved``: the rotation pairs
    neighbouring features (2i, 2i + 1) instead of (i, i + rot_dims/2)."""
    ld = _ld(qkv, "qkv")
    n = qkv.shape[0]
    if qkv.shape[1] < nh * dk + (nkv * (dk + dv) if write_kv else 0):
        raise KernelError(f"qkv_rotate_store: rows of {qkv.shape[1]} cannot hold {nh} query heads and {nkv} key/value heads")
    _need(q_out, "qkv q_out", qkv.dtype, (n, nh * dk))
    _need(positions, "qkv positions", torch.int32, (n,))
    if rot_dims:
        _need(inv_freq, "qkv inv_freq", torch.float32, (rot_dims // 2,))
    tw = pk = pv = 0
    if write_kv:
        _need(tok_slot, "qkv token slots", torch.int32, (n,))
        _need(page_table, "qkv page table", torch.int32, (None, None))
        _need(kpool, "qkv key pool", qkv.dtype, (None, page_size, None))
        _need(vpool, "qkv value pool", qkv.dtype, (kpool.shape[0], page_size, None))
        if kpool.shape[2] % nkv or vpool.shape[2] % nkv:
            raise KernelError(f"qkv_rotate_store: pools of {kpool.shape[2]} / {vpool.shape[2]} features do not hold {nkv} heads")
        tw, pk, pv = page_table.shape[1], kpool.shape[2] // nkv, vpool.shape[2] // nkv
    _check(_fn("attention_general", "cpmcu_qkv_rotate_store")(
        _p(qkv), c_long(ld), c_int(_code(qkv)), _p(q_out), c_int(n), c_int(nh), c_int(nkv), c_int(dk), c_int(dv),
        c_int(rot_dims), _p(positions), _p(tok_slot), _p(inv_freq), c_float(mag), _p(kpool if write_kv else None),
        _p(vpool if write_kv else None), _p(page_table if write_kv else None), c_int(tw), c_int(page_size), c_int(pk),
        c_int(pv), c_int(1 if write_kv else 0), c_int(1 if interleaved else 0), _stream()))


def qkv_norm_rotate_store(qkv: torch.Tensor, q_out: torch.Tensor, nh: int, nkv: int, dk: int, dv: int, rot_dims: int,
                          positions: torch.Tensor, tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mag: float,
                          kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor],
                          page_table: Optional[torch.Tensor], page_size: int, write_kv: bool = True,
                          bias: Optional[torch.Tensor] = None, q_norm: Optional[torch.Tensor] = None,
                          k_norm: Optional[torch.Tensor] = None, eps: float = 0.0, values_from_keys: bool = False,
                          norm_after: bool = False, interleaved: bool = False):
    """qkv_rotate_store with what some designs put between projection and rotation: ``bias`` (float32, as wide as
    a row of qkv) is added; q heads and k heads are divided by their root mean square (eps inside the root) and
    multiplied by a weight of dk numbers shared by the heads (q_norm, k_norm, float32 [dk]); with
    values_from_keys a row is [q | k] only and the value pages receive k as projected (with its bias, before norm
    and rotation).  With norm_after the q and k heads are rotated first and then divided by their root mean square
    (times q_norm / k_norm where given, by nothing else where not).  ``interleaved`` as in qkv_rotate_store.  The
    rows of qkv may be float32 where q_out and the cache are bfloat16 (rows that a convolution wrote)."""
    ld = _ld(qkv, "qkv")
    n = qkv.shape[0]
    width = nh * dk + ((nkv * dk + (0 if values_from_keys else nkv * dv)) if write_kv else 0)
    if qkv.shape[1] < width:
        raise KernelError(f"qkv_norm_rotate_store: rows of {qkv.shape[1]} cannot hold {nh} query heads and {nkv} key/value heads")
    if values_from_keys and dv != dk:
        raise KernelError(f"qkv_norm_rotate_store: values that are the keys have the keys' size ({dv}, {dk})")
    _need(q_out, "qkv q_out", shape=(n, nh * dk))
    if qkv.dtype != q_out.dtype and qkv.dtype != torch.float32:
        raise KernelError(f"qkv_norm_rotate_store: rows of {qkv.dtype} for outputs of {q_out.dtype}")
    _need(positions, "qkv positions", torch.int32, (n,))
    if rot_dims:
        _need(inv_freq, "qkv inv_freq", torch.float32, (rot_dims // 2,))
    if bias is not None:
        _need(bias, "qkv bias", torch.float32, (None,))
        if bias.shape[0] < width:
            raise KernelError(f"qkv_norm_rotate_store: a bias of {bias.shape[0]} numbers for rows of {width}")
    for t, name in ((q_norm, "query norm weight"), (k_norm, "key norm weight")):
        if t is not None:
            _need(t, f"qkv {name}", torch.float32, (dk,))
    tw = pk = pv = 0
    if write_kv:
        _need(tok_slot, "qkv token slots", torch.int32, (n,))
        _need(page_table, "qkv page table", torch.int32, (None, None))
        _need(kpool, "qkv key pool", q_out.dtype, (None, page_size, None))
        _need(vpool, "qkv value pool", q_out.dtype, (kpool.shape[0], page_size, None))
        if kpool.shape[2] % nkv or vpool.shape[2] % nkv:
            raise KernelError(f"qkv_norm_rotate_store: pools of {kpool.shape[2]} / {vpool.shape[2]} features do not hold {nkv} heads")
        tw, pk, pv = page_table.shape[1], kpool.shape[2] // nkv, vpool.shape[2] // nkv
    _check(_fn("attention_general", "cpmcu_qkv_norm_rotate_store")(
        _p(qkv), c_long(ld), c_int(_code(q_out)), _p(bias), _p(q_out), c_int(n), c_int(nh), c_int(nkv), c_int(dk), c_int(dv),
        c_int(rot_dims), _p(q_norm), _p(k_norm), c_float(eps), c_int(1 if values_from_keys else 0), _p(positions),
        _p(tok_slot), _p(inv_freq), c_float(mag), _p(kpool if write_kv else None), _p(vpool if write_kv else None),
        _p(page_table if write_kv else None), c_int(tw), c_int(page_size), c_int(pk), c_int(pv),
        c_int(1 if write_kv else 0), c_int(1 if norm_after else 0), c_int(1 if interleaved else 0), c_int(_code(qkv)),
        _stream()))


def _parts_of(t: torch.Tensor, n: int, H: int, name: str):
    """(parts, stride) of a branch [n, H] or of float partial sums [P, n, H]."""
    if t.dim() == 3:
        _need(t, name, shape=(None, n, H))
        return t.shape[0], n * H
    _need(t, name, shape=(n, H))
    return 1, 0


def gated_branches(gates: torch.Tensor, gate_bias: Optional[torch.Tensor], a: torch.Tensor, a_bias: Optional[torch.Tensor],
                   f: Optional[torch.Tensor], f_bias: Optional[torch.Tensor], out: torch.Tensor):
    """out = sigmoid(gates[:, :H] + gate_bias[:H]) * (a + a_bias) + sigmoid(gates[:, H:2H] + gate_bias[H:]) * (f + f_bias),
    in float; a and f [n, H] or float partial sums [P, n, H]; f (with its gate) may be None.  gates may be a column
    slice of a wider projection."""
    _need(out, "gated out", torch.float32, (None, None))
    n, H = out.shape
    ldg = _ld(gates, "gates")
    if gates.shape[0] != n or gates.shape[1] < (2 if f is not None else 1) * H:
        raise KernelError(f"gated_branches: gates {tuple(gates.shape)} for {n} rows of {H}")
    ap, astr = _parts_of(a, n, H, "gated branch")
    fp, fstr = _parts_of(f, n, H, "gated second branch") if f is not None else (0, 0)
    if gate_bias is not None:
        _need(gate_bias, "gate bias", torch.float32, ((2 if f is not None else 1) * H,))
    for t, name in ((a_bias, "branch bias"), (f_bias, "second branch bias")):
        if t is not None:
            _need(t, name, torch.float32, (H,))
    _check(_fn("norms", "cpmcu_gated_branches")(
        _p(gates), c_long(ldg), c_int(_code(gates)), _p(gate_bias), _p(a), c_int(_code(a)), c_int(ap), c_long(astr),
        _p(a_bias), _p(f), c_int(_code(f) if f is not None else 0), c_int(fp), c_long(fstr), _p(f_bias), _p(out),
        c_int(n), c_int(H), _stream()))


def bias_sum(a: torch.Tensor, bias: torch.Tensor, out: torch.Tensor):
    """out = a + bias in float, a [n, H] or float partial sums [P, n, H] (summed)."""
    _need(out, "bias_sum out", torch.float32, (None, None))
    n, H = out.shape
    parts, stride = _parts_of(a, n, H, "bias_sum input")
    _need(bias, "bias", torch.float32, (H,))
    _check(_fn("norms", "cpmcu_bias_sum")(_p(a), c_int(_code(a)), c_int(parts), c_long(stride), _p(bias), _p(out),
                                          c_int(n), c_int(H), _stream()))


def scaled_branches(a: torch.Tensor, a_bias: Optional[torch.Tensor], a_weight: Optional[torch.Tensor], a_scale: float,
                    f: Optional[torch.Tensor], f_bias: Optional[torch.Tensor], f_weight: Optional[torch.Tensor],
                    f_scale: float, out: torch.Tensor):
    """out = a_scale * a_weight * (a + a_bias) + f_scale * f_weight * (f + f_bias) in float: a and f [n, H] or float
    partial sums [P, n, H]; the weights (float32 [H], a number a column) and biases may be None, and so may f."""
    _need(out, "scaled out", torch.float32, (None, None))
    n, H = out.shape
    ap, astr = _parts_of(a, n, H, "scaled branch")
    fp, fstr = _parts_of(f, n, H, "scaled second branch") if f is not None else (0, 0)
    for t, name in ((a_bias, "branch bias"), (f_bias, "second branch bias"), (a_weight, "branch weight"),
                    (f_weight, "second branch weight")):
        if t is not None:
            _need(t, name, torch.float32, (H,))
    _check(_fn("norms", "cpmcu_scaled_branches")(
        _p(a), c_int(_code(a)), c_int(ap), c_long(astr), _p(a_bias), _p(a_weight), c_float(a_scale), _p(f),
        c_int(_code(f) if f is not None else 0), c_int(fp), c_long(fstr), _p(f_bias), _p(f_weight), c_float(f_scale),
        _p(out), c_int(n), c_int(H), _stream()))


def bigram_add(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, tok_slot: torch.Tensor,
               prev_state: torch.Tensor, cu_q: torch.Tensor, seq_slot: torch.Tensor, out: torch.Tensor, buckets: int,
               mul_prev: int, mul_cur: int, remember: bool = True):
    """out[r] += float(table[(prev * mul_prev + ids[r] * mul_cur) % buckets]); a token at position 0 reads row
    ``buckets`` (the last of the table's buckets + 1 rows).  prev is the token before it in its sequence: the row
    above in the packed batch, or, for the first row a sequence brings, prev_state[slot] (int32 [slots]).  With
    ``remember`` every sequence's slot then holds the last token it brought."""
    _need(table, "bigram table", shape=(buckets + 1, None))
    H = table.shape[1]
    _need(ids, "bigram ids", torch.int32, (None,))
    n = ids.shape[0]
    _need(positions, "bigram positions", torch.int32, (n,))
    _need(tok_slot, "bigram token slots", torch.int32, (n,))
    _need(prev_state, "bigram previous tokens", torch.int32, (None,))
    _need(cu_q, "bigram sequence starts", torch.int32, (None,))
    B = cu_q.shape[0] - 1
    _need(seq_slot, "bigram sequence slots", torch.int32, (B,))
    _need(out, "bigram out", torch.float32, (n, H))
    if buckets <= 0 or mul_prev < 0 or mul_cur < 0:
        raise KernelError(f"bigram_add: {buckets} buckets, multipliers {mul_prev}, {mul_cur}")
    _check(_fn("core", "cpmcu_bigram_add")(_p(table), c_int(_code(table)), _p(ids), _p(positions), _p(tok_slot),
                                           _p(prev_state), _p(cu_q), _p(seq_slot), _p(out), c_int(n), c_int(B), c_int(H),
                                           c_long(buckets), c_long(mul_prev), c_long(mul_cur),
                                           c_int(1 if remember else 0), _stream()))


def mlstm_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, i_off: int, f_off: int, i_bias: torch.Tensor,
               f_bias: torch.Tensor, cap: float, q_scale: float, S: torch.Tensor, n_state: torch.Tensor,
               m_state: torch.Tensor, y: torch.Tensor, den: torch.Tensor, cu_q: torch.Tensor, seq_slot: torch.Tensor,
               heads: int, d: int, dv: int, write_state: bool = True):
    """The matrix-memory recurrence over each sequence's tokens, in float.  proj [n, W] holds, from the given
    columns on, q and k (heads * d each), v (heads * dv) and the raw input and forget gates (heads each); per head
    a = cap tanh((i + i_bias)/cap), b = logsigmoid(cap tanh((f + f_bias)/cap)), m' = max(b + m, a),
    S' = exp(b + m - m') S + exp(a - m') k v^T, n' likewise with k, q multiplied by q_scale.  It leaves the output
    in two pieces: y = S'^T q (float32 [n, heads * dv]) and den = max(|n'.q|, exp(-m')) + 1e-6 (float32 [n, heads]);
    the design's output is y / den head by head (rms_norm_groups takes den as its divisor).
    S float32 [slots, heads, dv, d], n_state [slots, heads, d], m_state [slots, heads]."""
    ld = _ld(proj, "mlstm projection")
    n = proj.shape[0]
    for off, w in ((q_off, heads * d), (k_off, heads * d), (v_off, heads * dv), (i_off, heads), (f_off, heads)):
        if off < 0 or off + w > proj.shape[1]:
            raise KernelError(f"mlstm_scan: columns {off}..{off + w} lie beyond rows of {proj.shape[1]}")
    _need(i_bias, "mlstm input gate bias", torch.float32, (heads,))
    _need(f_bias, "mlstm forget gate bias", torch.float32, (heads,))
    _need(S, "mlstm state", torch.float32, (None, heads, dv, d))
    _need(n_state, "mlstm normaliser", torch.float32, (S.shape[0], heads, d))
    _need(m_state, "mlstm maximum", torch.float32, (S.shape[0], heads))
    _need(y, "mlstm out", torch.float32, (n, heads * dv))
    _need(den, "mlstm denominators", torch.float32, (n, heads))
    _need(cu_q, "mlstm sequence starts", torch.int32, (None,))
    B = cu_q.shape[0] - 1
    _need(seq_slot, "mlstm sequence slots", torch.int32, (B,))
    _check(_fn("mlstm", "cpmcu_mlstm_scan")(_p(proj), c_long(ld), c_int(_code(proj)), c_long(q_off), c_long(k_off),
                                            c_long(v_off), c_long(i_off), c_long(f_off), _p(i_bias), _p(f_bias),
                                            c_float(cap), c_float(q_scale), _p(S), _p(n_state), _p(m_state), _p(y),
                                            _p(den), _p(cu_q), _p(seq_slot), c_int(B), c_int(heads), c_int(d), c_int(dv),
                                            c_int(1 if write_state else 0), _stream()))


def streams_fill(x: torch.Tensor, streams: torch.Tensor):
    """streams[s] = x for every s: a residual of several streams starts as copies of the embedding's output.
    x float32 [n, H], streams float32 [S, n, H]."""
    _need(x, "streams source", torch.float32, (None, None))
    n, H = x.shape
    _need(streams, "residual streams", torch.float32, (None, n, H))
    _check(_fn("norms", "cpmcu_streams_fill")(_p(x), _p(streams), c_long(n * H), c_int(streams.shape[0]), _stream()))


def streams_norm(x: torch.Tensor, branch: Optional[torch.Tensor], branch_bias: Optional[torch.Tensor],
                 branch_scale: float, mix: Optional[torch.Tensor], out_weights: Optional[torch.Tensor],
                 read: Optional[torch.Tensor], weight: torch.Tensor, eps: float, out: torch.Tensor,
                 rows: Optional[torch.Tensor] = None, rms: bool = False):
    """The residual add and the norm that follows it, for a residual of S >= 1 streams x float32 [S, n, H] (or
    [n, H], one stream).  With a branch y = branch_scale * branch (+ branch_bias; summed over the leading axis if
    it is [P, n, H]):  x_t <- sum_s mix[s, t] x_s + out_weights[t] * y  (mix float32 [S, S] indexed [from, to],
    None: each stream keeps itself; out_weights float32 [S], None: ones), all streams at once, in place.  Then
    u = sum_t read[t] x_t (read float32 [S], None: the plain sum) and out = layer norm without bias of u,
    (u - mean) / sqrt(variance + eps) * weight, or with ``rms`` u / sqrt(mean(u^2) + eps) * weight.  With ``rows``
    (int32 [R]) only those rows are computed, into out [R, H], and x is left as it was."""
    if x.dim() == 2:
        _need(x, "residual", torch.float32, (None, None))
        S, (n, H) = 1, x.shape
    else:
        _need(x, "residual streams", torch.float32, (None, None, None))
        S, n, H = x.shape
    _need(weight, "norm weight", torch.float32, (H,))
    nparts, stride, bcode = 1, 0, F32
    if branch is not None:
        nparts, stride = _parts_of(branch, n, H, "norm branch")
        bcode = _code(branch)
        if branch_bias is not None:
            _need(branch_bias, "branch bias", torch.float32, (H,))
    elif mix is not None or out_weights is not None:
        raise KernelError("streams_norm: mixing numbers without a branch to add")
    if mix is not None:
        _need(mix, "stream mix", torch.float32, (S, S))
    for t, name in ((out_weights, "stream out weights"), (read, "stream read weights")):
        if t is not None:
            _need(t, name, torch.float32, (S,))
    n_out = n
    if rows is not None:
        _need(rows, "norm rows", torch.int32, (None,))
        n_out = rows.shape[0]
    _need(out, "norm out", shape=(n_out, H))
    _check(_fn("norms", "cpmcu_streams_norm")(
        _p(x), c_long(n * H), c_int(S), _p(branch), c_int(bcode), c_int(nparts), c_long(stride),
        _p(branch_bias if branch is not None else None), c_float(branch_scale), _p(mix), _p(out_weights), _p(read),
        c_int(1 if rms else 0), _p(weight), c_float(eps), _p(out), c_int(_code(out)), _p(rows), c_int(n_out), c_int(H),
        _stream()))


def pair_norm_mean(a: torch.Tensor, a_bias: Optional[torch.Tensor], b: torch.Tensor, b_bias: Optional[torch.Tensor],
                   wa: torch.Tensor, wb: torch.Tensor, eps: float, out: torch.Tensor):
    """out = (a / rms(a) * wa + b / rms(b) * wb) / 2 row by row in float, rms(v) = sqrt(mean(v^2) + eps): the
    results of two mixers side by side.  a and b [n, H] or float partial sums [P, n, H], each with an optional
    bias float32 [H] still to be added."""
    _need(out, "pair out", torch.float32, (None, None))
    n, H = out.shape
    ap, astr = _parts_of(a, n, H, "pair first branch")
    bp, bstr = _parts_of(b, n, H, "pair second branch")
    for t, name in ((wa, "first weight"), (wb, "second weight"), (a_bias, "first bias"), (b_bias, "second bias")):
        if t is not None:
            _need(t, f"pair {name}", torch.float32, (H,))
    _check(_fn("norms", "cpmcu_pair_norm_mean")(_p(a), c_int(_code(a)), c_int(ap), c_long(astr), _p(a_bias), _p(b),
                                                c_int(_code(b)), c_int(bp), c_long(bstr), _p(b_bias), _p(wa), _p(wb),
                                                c_float(eps), _p(out), c_int(n), c_int(H), _stream()))


def sigmoid_gate(a: torch.Tensor, gate: torch.Tensor, out: torch.Tensor):
    """out = a * sigmoid(gate) element by element; gate may be a column slice of a wider projection."""
    _need(a, "gate input", shape=(None, None))
    n, W = a.shape
    ldg = _ld(gate, "gate")
    if gate.dtype != a.dtype or tuple(gate.shape) != (n, W):
        raise KernelError(f"sigmoid_gate: gate {gate.dtype} {tuple(gate.shape)}, expected {a.dtype} {(n, W)}")
    _need(out, "gate out", a.dtype, (n, W))
    _check(_fn("norms", "cpmcu_sigmoid_gate")(_p(a), _p(gate), c_long(ldg), _p(out), c_int(_code(a)), c_int(n), c_int(W),
                                              _stream()))


def softcap(logits: torch.Tensor, cap: float):
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _need(logits, "softcap logits", torch.float32)
    if not cap > 0:
        raise KernelError(f"softcap: a cap of {cap}")
    _check(_fn("core", "cpmcu_softcap")(_p(logits), c_long(logits.numel()), c_float(cap), _stream()))


def delta_scan(qkv: torch.Tensor, gates: Optional[torch.Tensor], a_off: int, b_off: int, dt_bias: Optional[torch.Tensor],
               A_log: torch.Tensor, state: torch.Tensor, y: torch.Tensor, cu_q: torch.Tensor, seq_slot: torch.Tensor,
               heads: int, kv_heads: int, dk: int, dv: int, q_scale: float, write_state: bool = True, lanes: int = 0,
               rule: str = "delta", channel_decay: Optional[torch.Tensor] = None):
    """The gated delta rule over each sequence's tokens, in float.  qkv float32 [n, 2*kv_heads*dk + heads*dv] =
    [q | k | v]; gates [n, W] holds the raw decay projection at columns a_off.. and the raw beta projection at
    b_off.. (heads each).  Per head (its q, k from head h // (heads/kv_heads)): q, k made unit vectors
    (x / sqrt(sum x^2 + 1e-6)), q times q_scale; beta = sigmoid(b); g = exp(-exp(A_log) softplus(a + dt_bias));
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; y = S^T q.  state float32 [slots, heads, dv, dk]; y float32
    [n, heads*dv].  lanes: how many lanes share a column of the state (8 or 16; 0: chosen by how much the batch
    gives the chip to do).
    rule 'channel': the decay is a number a head and key channel, S <- diag(g) S with g = exp(-exp(A_log[h])
    softplus(channel_decay[:, h*dk + i] + dt_bias[h*dk + i])); channel_decay float32 [n, heads*dk] (may be a column
    slice), dt_bias float32 [heads*dk]; a_off is not read.
    rule 'decay': linear attention with a fixed decay a head, S <- A_log[h] S + k v^T, y = S^T q, q and k as they
    come; no gates, no dt_bias (A_log holds the decays themselves)."""
    if rule not in DELTA_RULES:
        raise KernelError(f"delta_scan: rule '{rule}' ({sorted(DELTA_RULES)})")
    _need(qkv, "delta inputs", torch.float32, (None, 2 * kv_heads * dk + heads * dv))
    n = qkv.shape[0]
    ldg = ld_a = 0
    if rule != "decay":
        ldg = _ld(gates, "delta gates")
        cols = (b_off,) if rule == "channel" else (a_off, b_off)
        if gates.shape[0] != n or min(cols) < 0 or max(cols) + heads > gates.shape[1]:
            raise KernelError(f"delta_scan: gate columns {cols} (+{heads}) lie beyond rows of {tuple(gates.shape)}")
        _need(dt_bias, "delta dt_bias", torch.float32, (heads * dk if rule == "channel" else heads,))
    if rule == "channel":
        ld_a = _ld(channel_decay, "delta channel decay")
        if channel_decay.dtype != torch.float32 or tuple(channel_decay.shape) != (n, heads * dk):
            raise KernelError(f"delta_scan: channel decay {channel_decay.dtype} {tuple(channel_decay.shape)}, expected "
                              f"float32 {(n, heads * dk)}")
    _need(A_log, "delta A_log", torch.float32, (heads,))
    _need(state, "delta state", torch.float32, (None, heads, dv, dk))
    _need(y, "delta out", torch.float32, (n, heads * dv))
    _need(cu_q, "delta sequence starts", torch.int32, (None,))
    B = cu_q.shape[0] - 1
    _need(seq_slot, "delta sequence slots", torch.int32, (B,))
    _check(_fn("delta", "cpmcu_delta_scan")(_p(qkv), c_long(qkv.shape[1]), _p(gates), c_long(ldg),
                                            c_int(_code(gates) if gates is not None else 0), c_long(a_off), c_long(b_off),
                                            _p(channel_decay), c_long(ld_a), _p(dt_bias), _p(A_log), _p(state), _p(y),
                                            _p(cu_q), _p(seq_slot), c_int(B), c_int(heads), c_int(kv_heads), c_int(dk),
                                            c_int(dv), c_float(q_scale), c_int(1 if write_state else 0), c_int(lanes),
                                            c_int(DELTA_RULES[rule]), _stream()))


DELTA_RULES = {"delta": 0, "channel": 1, "decay": 2}


def linear_attention_prepare(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, out: torch.Tensor, heads: int,
                             dk: int, dv: int, silu: bool, positions: Optional[torch.Tensor] = None,
                             inv_freq: Optional[torch.Tensor] = None, interleaved: bool = False, k_scale: float = 1.0):
    """What linear attention puts between its projection and its recurrence, in float: proj [n, W] holds q heads at
    column q_off and k heads at k_off (heads x dk each) and v heads at v_off (heads x dv); out float32
    [n, 2*heads*dk + heads*dv] = [q | k | v].  With silu all three pass z sigmoid(z); with inv_freq (float32
    [r/2]) the first r features of q and k heads are rotated by positions * inv_freq (pairs (i, i + r/2), or
    neighbours when interleaved); k is multiplied by k_scale."""
    ld = _ld(proj, "linear attention projection")
    n = proj.shape[0]
    if min(q_off, k_off, v_off) < 0 or max(q_off + heads * dk, k_off + heads * dk, v_off + heads * dv) > proj.shape[1]:
        raise KernelError(f"linear_attention_prepare: columns beyond rows of {tuple(proj.shape)}")
    _need(out, "linear attention inputs", torch.float32, (n, 2 * heads * dk + heads * dv))
    rot = 0
    if inv_freq is not None:
        _need(inv_freq, "linear attention inv_freq", torch.float32, (None,))
        rot = 2 * inv_freq.shape[0]
        _need(positions, "linear attention positions", torch.int32, (n,))
        if rot > dk:
            raise KernelError(f"linear_attention_prepare: the rotation covers {rot} features, a head has {dk}")
    _check(_fn("delta", "cpmcu_linear_attention_prepare")(
        _p(proj), c_int(_code(proj)), c_long(ld), c_long(q_off), c_long(k_off), c_long(v_off), _p(out), c_int(n),
        c_int(heads), c_int(dk), c_int(dv), c_int(1 if silu else 0), c_int(rot), c_int(1 if interleaved else 0),
        _p(inv_freq), _p(positions), c_float(k_scale), _stream()))


def diff_qkv_store(src: torch.Tensor, q_out: torch.Tensor, heads: int, kv_heads: int, dk: int, dv: int,
                   temp_coef: float, temp_every: int, positions: torch.Tensor, tok_slot: torch.Tensor,
                   kpool: Optional[torch.Tensor], vpool: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
                   page_size: int, write_kv: bool = True):
    """Between projection and attention of a layer with two score maps a head: a row of src (float32 or q_out's
    type) is [q: heads*2*dk | k: kv_heads*2*dk | v: kv_heads*dv], q and k head by head as [map 1 | map 2].  q times
    1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) (temp_every 0: times 1) goes to q_out [n, 2*heads*dk] in
    the order (kv head, map, head of the group); k into the key pages as 2*kv_heads heads, v into the value pages
    as kv_heads heads."""
    ld = _ld(src, "diff qkv")
    n = src.shape[0]
    if src.shape[1] < 2 * heads * dk + ((2 * kv_heads * dk + kv_heads * dv) if write_kv else 0):
        raise KernelError(f"diff_qkv_store: rows of {src.shape[1]} too short")
    _need(q_out, "diff q_out", shape=(n, 2 * heads * dk))
    _need(positions, "diff positions", torch.int32, (n,))
    tw = pk = pv = 0
    if write_kv:
        _need(tok_slot, "diff token slots", torch.int32, (n,))
        _need(page_table, "diff page table", torch.int32, (None, None))
        _need(kpool, "diff key pool", q_out.dtype, (None, page_size, None))
        _need(vpool, "diff value pool", q_out.dtype, (kpool.shape[0], page_size, None))
        if kpool.shape[2] % (2 * kv_heads) or vpool.shape[2] % kv_heads:
            raise KernelError(f"diff_qkv_store: pools of {kpool.shape[2]} / {vpool.shape[2]} features")
        tw, pk, pv = page_table.shape[1], kpool.shape[2] // (2 * kv_heads), vpool.shape[2] // kv_heads
    _check(_fn("attention_general", "cpmcu_diff_qkv_store")(
        _p(src), c_long(ld), c_int(_code(src)), _p(q_out), c_int(_code(q_out)), c_int(n), c_int(heads), c_int(kv_heads),
        c_int(dk), c_int(dv), c_float(temp_coef), c_int(temp_every), _p(positions), _p(tok_slot),
        _p(kpool if write_kv else None), _p(vpool if write_kv else None), _p(page_table if write_kv else None),
        c_int(tw), c_int(page_size), c_int(pk), c_int(pv), c_int(1 if write_kv else 0), _stream()))


def diff_combine(a: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int, dv: int, lam: float, eps: float,
                 post: float):
    """out[t, h] = o / sqrt(mean(o^2) + eps) * post with o = a1 - lam * a2, the two maps' attention outputs of head
    h; a [n, 2*heads*dv] in the order (kv head, map, head of the group; float32, or out's type), out [n, heads*dv]."""
    _need(a, "diff maps", shape=(None, 2 * heads * dv))
    n = a.shape[0]
    _need(out, "diff out", shape=(n, heads * dv))
    _check(_fn("attention_general", "cpmcu_diff_combine")(_p(a), c_int(_code(a)), _p(out), c_int(_code(out)), c_int(n), c_int(heads),
                                                          c_int(kv_heads), c_int(dv), c_float(lam), c_float(eps),
                                                          c_float(post), _stream()))


MOE_MAX_EXPERTS = 1024
MOE_SCORES = {"softmax": 0, "sigmoid": 1}
MOE_GROUP_SCORES = {"max": 0, "top2_sum": 1}


def moe_route(h: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor],
              n_groups: int, keep_groups: int, top: int, idx: torch.Tensor, weights: torch.Tensor,
              shared_out: Optional[torch.Tensor] = None, logits: Optional[torch.Tensor] = None,
              score: str = "softmax", group_score: str = "max", weight_scale: float = 1.0):
    """Routing of every token to ``top`` of E experts.  Logits router . h in float (router float32 [E, H]), scores
    s = softmax over the experts (``score`` 'sigmoid': of each logit alone); choice scores s + correction; the
    experts form n_groups equal groups of neighbours, of which only the keep_groups with the largest group score may
    be chosen from (``group_score`` 'max': a group's best choice score; 'top2_sum': the sum of its two best); the top
    largest choice scores win (ties: the lower index); weights = s of the chosen / (their sum + 1e-20) *
    weight_scale.  idx int32 [n, top], weights float32 [n, top].
    shared_gate (float32 [H]): shared_out[t] = sigmoid(shared_gate . h[t]).  logits: float32 [n, E + 1] of scratch
    (allocated here when absent: a caller that must not allocate brings it)."""
    ldh = _ld(h, "router input")
    n, H = h.shape
    _need(router, "router weight", torch.float32, (None, H))
    E = router.shape[0]
    if correction is not None:
        _need(correction, "router correction", torch.float32, (E,))
    if shared_gate is not None:
        _need(shared_gate, "shared gate weight", torch.float32, (H,))
        _need(shared_out, "shared gate", torch.float32, (n,))
    _need(idx, "chosen experts", torch.int32, (n, top))
    _need(weights, "expert weights", torch.float32, (n, top))
    if logits is None:
        logits = torch.empty((n, E + 1), dtype=torch.float32, device=h.device)
    _need(logits, "router logits", torch.float32, (n, E + 1))
    if score not in MOE_SCORES or group_score not in MOE_GROUP_SCORES:
        raise KernelError(f"moe_route: score '{score}' ({sorted(MOE_SCORES)}) or group score '{group_score}' "
                          f"({sorted(MOE_GROUP_SCORES)}) is not known")
    _check(_fn("moe", "cpmcu_moe_route")(_p(h), c_long(ldh), c_int(_code(h)), _p(router), _p(correction), _p(shared_gate),
                                         c_int(n), c_int(H), c_int(E), c_int(n_groups), c_int(keep_groups), c_int(top),
                                         _p(logits), _p(idx), _p(weights), _p(shared_out), c_int(MOE_SCORES[score]),
                                         c_int(MOE_GROUP_SCORES[group_score]), c_float(weight_scale), _stream()))


def moe_gated(h: torch.Tensor, gate_up: torch.Tensor, idx: torch.Tensor, act: torch.Tensor, activation="silu"):
    """act[t, k] = act(Wg_e h[t]) * (Wu_e h[t]) for e = idx[t, k] (act: SiLU, or as gate_activation says); gate_up
    [E, 2F, H] (an expert's gate rows, then its up rows), act [n, top, F], both of h's element type."""
    ldh = _ld(h, "experts input")
    n, H = h.shape
    _need(gate_up, "experts gate/up", h.dtype, (None, None, H))
    E, F2 = gate_up.shape[0], gate_up.shape[1]
    if F2 % 2:
        raise KernelError(f"moe_gated: {F2} stacked gate and up rows")
    _need(idx, "chosen experts", torch.int32, (n, None))
    top = idx.shape[1]
    _need(act, "experts act", h.dtype, (n, top, F2 // 2))
    _check(_fn("moe", "cpmcu_moe_gated")(_p(h), c_long(ldh), c_int(_code(h)), _p(gate_up), _p(idx), _p(act), c_int(n),
                                         c_int(H), c_int(F2 // 2), c_int(top), *_act(activation), _stream()))


def moe_down(act: torch.Tensor, down: torch.Tensor, idx: torch.Tensor, weights: torch.Tensor, out: torch.Tensor,
             shared: Optional[torch.Tensor] = None, shared_gate: Optional[torch.Tensor] = None):
    """out[t] = sum_k weights[t, k] * Wd_e act[t, k] (+ shared_gate[t] * shared[t]); down [E, H, F]; out float32
    [n, H]; shared [n, H] or float partial sums [P, n, H]."""
    _need(act, "experts act", shape=(None, None, None))
    n, top, F = act.shape
    _need(down, "experts down", act.dtype, (None, None, F))
    H = down.shape[1]
    _need(idx, "chosen experts", torch.int32, (n, top))
    _need(weights, "expert weights", torch.float32, (n, top))
    _need(out, "experts out", torch.float32, (n, H))
    sp, sstr = _parts_of(shared, n, H, "shared expert") if shared is not None else (0, 0)
    if shared_gate is not None:
        _need(shared_gate, "shared gate", torch.float32, (n,))
    _check(_fn("moe", "cpmcu_moe_down")(_p(act), c_int(_code(act)), _p(down), _p(idx), _p(weights), _p(shared),
                                        c_int(_code(shared) if shared is not None else 0), c_int(sp), c_long(sstr),
                                        _p(shared_gate), _p(out), c_int(n), c_int(H), c_int(F), c_int(top), _stream()))


MOE_TILE = 64


def moe_tiles(n: int, top: int, experts: int) -> int:
    """Tiles of MOE_TILE rows that moe_experts_mfma's scratch must hold for n tokens: every expert's pairs fill whole
    tiles, so up to one tile an expert is partly empty."""
    return -(-(n * top) // MOE_TILE) + experts


def moe_experts_mfma_ok(h: torch.Tensor, expert_size: int, n_tiles: int) -> bool:
    return (h.dtype == torch.bfloat16 and h.shape[1] % 8 == 0 and expert_size % 8 == 0 and n_tiles <= 65535
            and h.stride(0) % 8 == 0)


def moe_experts_mfma(h: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, idx: torch.Tensor, weights: torch.Tensor,
                     out: torch.Tensor, act: torch.Tensor, y: torch.Tensor, rows: torch.Tensor, tile_expert: torch.Tensor,
                     n_tiles: torch.Tensor, shared: Optional[torch.Tensor] = None,
                     shared_gate: Optional[torch.Tensor] = None, activation="silu"):
    """moe_gated + moe_down for steps of many tokens, bf16 on the matrix cores: the (token, expert) pairs are grouped
    by expert into tiles of MOE_TILE rows.  Scratch: act bf16 [n, top, F], y bf16 [n, top, H], rows int32
    [tiles * MOE_TILE], tile_expert int32 [tiles], n_tiles int32 [1], tiles >= moe_tiles(n, top, E)."""
    ldh = _ld(h, "experts input")
    n, H = h.shape
    _need(gate_up, "experts gate/up", torch.bfloat16, (None, None, H))
    E, F = gate_up.shape[0], gate_up.shape[1] // 2
    _need(down, "experts down", torch.bfloat16, (E, H, F))
    _need(idx, "chosen experts", torch.int32, (n, None))
    top = idx.shape[1]
    _need(weights, "expert weights", torch.float32, (n, top))
    _need(out, "experts out", torch.float32, (n, H))
    _need(act, "experts act", torch.bfloat16, (n, top, F))
    _need(y, "experts pair outputs", torch.bfloat16, (n, top, H))
    _need(tile_expert, "experts tile map", torch.int32, (None,))
    tiles = tile_expert.shape[0]
    _need(rows, "experts tile rows", torch.int32, (tiles * MOE_TILE,))
    _need(n_tiles, "experts tile count", torch.int32, (1,))
    if h.dtype != torch.bfloat16:
        raise KernelError("moe_experts_mfma: bfloat16 only")
    sp, sstr = _parts_of(shared, n, H, "shared expert") if shared is not None else (0, 0)
    if shared_gate is not None:
        _need(shared_gate, "shared gate", torch.float32, (n,))
    _check(_fn("moe", "cpmcu_moe_experts_mfma")(
        _p(h), c_long(ldh), _p(gate_up), _p(down), _p(idx), _p(weights), _p(shared),
        c_int(_code(shared) if shared is not None else 0), c_int(sp), c_long(sstr), _p(shared_gate), _p(act), _p(y),
        _p(rows), _p(tile_expert), _p(n_tiles), c_int(tiles), _p(out), c_int(n), c_int(H), c_int(F), c_int(E), c_int(top),
        *_act(activation), _stream()))


def latent_store(proj: torch.Tensor, q_out: torch.Tensor, nh: int, dim: int, rot: int, rank: int,
                 norm_w: Optional[torch.Tensor], eps: float, positions: torch.Tensor, tok_slot: torch.Tensor,
                 inv_freq: Optional[torch.Tensor], mag: float, kpool: Optional[torch.Tensor],
                 vpool: Optional[torch.Tensor], page_table: Optional[torch.Tensor], page_size: int,
                 write_cache: bool = True):
    """Latent attention's steps between projection and attention in one launch.  A row of proj is
    [nh heads of (dim plain | rot rotated) | rank + rot of the down projection (if write_cache) | ...]:
    every head's rotated part goes, rotated, to q_out[t, head, rank:rank+rot] (q_out [n, nh*(rank+rot)]); with
    write_cache the latent rmsnorm(down[:rank]) * norm_w goes into the key pages (features 0..rank) and the value
    pages, and down[rank:], rotated, into the key pages behind it."""
    ld = _ld(proj, "latent projection")
    n = proj.shape[0]
    if proj.shape[1] < nh * (dim + rot) + (rank + rot if write_cache else 0):
        raise KernelError(f"latent_store: rows of {proj.shape[1]} are too short")
    _need(q_out, "latent q_out", proj.dtype, (n, nh * (rank + rot)))
    _need(positions, "latent positions", torch.int32, (n,))
    if rot:
        _need(inv_freq, "latent inv_freq", torch.float32, (rot // 2,))
    tw = pk = pv = 0
    if write_cache:
        _need(norm_w, "latent norm weight", torch.float32, (rank,))
        _need(tok_slot, "latent token slots", torch.int32, (n,))
        _need(page_table, "latent page table", torch.int32, (None, None))
        _need(kpool, "latent key pool", proj.dtype, (None, page_size, None))
        _need(vpool, "latent value pool", proj.dtype, (kpool.shape[0], page_size, None))
        tw, pk, pv = page_table.shape[1], kpool.shape[2], vpool.shape[2]
    _check(_fn("attention_general", "cpmcu_latent_store")(
        _p(proj), c_long(ld), c_int(_code(proj)), _p(q_out), c_int(n), c_int(nh), c_int(dim), c_int(rot), c_int(rank),
        _p(norm_w if write_cache else None), c_float(eps), _p(positions), _p(tok_slot), _p(inv_freq), c_float(mag),
        _p(kpool if write_cache else None), _p(vpool if write_cache else None), _p(page_table if write_cache else None),
        c_int(tw), c_int(page_size), c_int(pk), c_int(pv), c_int(1 if write_cache else 0), _stream()))


def _value_heads(nkv: int, v_share: int) -> int:
    if v_share < 1 or nkv % v_share:
        raise KernelError(f"attention: {nkv} key heads do not share values in runs of {v_share}")
    return nkv // v_share


def attention_general(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hdk: int, hdv: int, scale: float,
                      kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                      positions: torch.Tensor, tok_slot: torch.Tensor, chunk: int = 0, window: int = 0,
                      keep_first: int = 0, sink: Optional[torch.Tensor] = None, v_share: int = 1,
                      softcap: float = 0.0):
    """Causal attention with key size hdk and value size hdv of their own (plain kernel, both element types).
    softcap c > 0: a scaled score s enters the softmax as c tanh(s / c).
    v_share: runs of that many neighbouring key heads read one value head (the value pool holds nkv / v_share heads).
    The cache may hold heads padded to a multiple of 16 features.  chunk > 0: the query at position p sees only
    keys j <= p with j // chunk == p // chunk.  window > 0: only keys with p - j < window, and the sequence's
    first keep_first keys.  sink (float32 [nh]): exp(sink[h]) joins the softmax's denominator as a term without
    a value."""
    if sink is not None:
        _need(sink, "attention sink", torch.float32, (nh,))
    _need(q, "attention q", shape=(None, nh * hdk))
    n = q.shape[0]
    _need(out, "attention out", q.dtype, (n, nh * hdv))
    _need(kpool, "attention key pool", q.dtype, (None, page_size, None))
    _need(vpool, "attention value pool", q.dtype, (kpool.shape[0], page_size, None))
    nvh = _value_heads(nkv, v_share)
    if kpool.shape[2] % nkv or vpool.shape[2] % nvh:
        raise KernelError(f"attention_general: pools of {kpool.shape[2]} / {vpool.shape[2]} features do not hold {nkv} / {nvh} heads")
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    _check(_fn("attention_general", "cpmcu_attention_general")(
        _p(q), _p(out), c_int(_code(q)), c_int(n), c_int(nh), c_int(nkv), c_int(hdk), c_int(hdv),
        c_int(kpool.shape[2] // nkv), c_int(vpool.shape[2] // nvh), c_float(scale), c_int(chunk), c_int(window),
        c_int(keep_first), _p(sink), _p(kpool),
        _p(vpool), _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot),
        c_int(v_share), c_float(softcap or 0.0), _stream()))


def gemm_heads(x: torch.Tensor, x_off: int, x_head_stride: int, w: torch.Tensor, out: torch.Tensor, out_off: int,
               out_head_stride: int, gate: Optional[torch.Tensor] = None, plain: bool = False):
    """out[m, out_off + h*out_head_stride + :N] = x[m, x_off + h*x_head_stride + :K] . w[h]^T for every head h;
    w [H, N, K].  With ``gate`` [m, H] head h's rows are multiplied by sigmoid(gate[m, h]).  bf16 runs on the
    matrix cores when K and the strides of x are multiples of 8 (``plain``: the scalar kernel all the same)."""
    ldx, ldy = _ld(x, "heads x"), _ld(out, "heads out")
    M = x.shape[0]
    _need(w, "heads weight", x.dtype, (None, None, None))
    H, N, K = w.shape
    if x_off < 0 or x_off + (H - 1) * x_head_stride + K > x.shape[1]:
        raise KernelError(f"gemm_heads: {H} heads of {K} features from column {x_off} do not fit rows of {x.shape[1]}")
    if out.shape[0] != M or out_off < 0 or out_off + (H - 1) * out_head_stride + N > out.shape[1]:
        raise KernelError(f"gemm_heads: {H} heads of {N} features to column {out_off} do not fit {tuple(out.shape)}")
    ldg = 0
    if gate is not None:
        ldg = _ld(gate, "heads gate")
        if gate.dtype != x.dtype or tuple(gate.shape) != (M, H):
            raise KernelError(f"heads gate: {gate.dtype} {tuple(gate.shape)}, expected {x.dtype} {(M, H)}")
    xp = c_void_p(x.data_ptr() + x_off * x.element_size())
    op = c_void_p(out.data_ptr() + out_off * out.element_size())
    if (x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and not plain and K % 8 == 0 and ldx % 8 == 0
            and x_head_stride % 8 == 0 and xp.value % 16 == 0 and w.data_ptr() % 16 == 0):
        _check(_fn("gemm", "cpmcu_gemm_nt_heads_mfma")(xp, c_long(ldx), c_long(x_head_stride), _p(w), op, c_long(ldy),
                                                       c_long(out_head_stride), _p(gate), c_long(ldg), c_int(M),
                                                       c_int(H), c_int(N), c_int(K), _stream()))
        return
    _check(_fn("gemm", "cpmcu_gemm_nt_heads")(xp, c_long(ldx), c_long(x_head_stride), _p(w), op, c_long(ldy),
                                              c_long(out_head_stride), _p(gate), c_long(ldg), c_int(_code(x)),
                                              c_int(_code(out)), c_int(M), c_int(H), c_int(N), c_int(K), _stream()))


def argmax(logits: torch.Tensor, out: torch.Tensor):
    """out[r] = index of the largest logits[r] (ties: the lowest index)."""
    _need(logits, "argmax logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(out, "argmax out", torch.int32, (R,))
    _check(_fn("core", "cpmcu_argmax")(_p(logits), c_long(V), c_int(R), c_int(V), _p(out), _stream()))


def sample(logits: torch.Tensor, temperature: float, seed: int, request_ids: torch.Tensor, steps: torch.Tensor,
           out: torch.Tensor, u_out: Optional[torch.Tensor] = None):
    """out[r] ~ softmax(logits[r] / temperature), the uniform number keyed by (seed, request_ids[r], steps[r])."""
    _need(logits, "sample logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(request_ids, "sample request ids", torch.int32, (R,))
    _need(steps, "sample steps", torch.int32, (R,))
    _need(out, "sample out", torch.int32, (R,))
    if u_out is not None:
        _need(u_out, "sample u_out", torch.float32, (R,))
    _check(_fn("core", "cpmcu_sample")(_p(logits), c_long(V), c_int(R), c_int(V), c_float(temperature),
                                       c_ulonglong(seed & 0xFFFFFFFFFFFFFFFF), _p(request_ids), _p(steps), _p(out),
                                       _p(u_out), _stream()))


def read_bandwidth(src: torch.Tensor, out: torch.Tensor):
    """Read all of ``src`` once with a kernel that does nothing else (out: int32 scratch of a few thousand
    words): what measurement compares the decode products' streaming with."""
    _need(src, "read source")
    _need(out, "read scratch", torch.int32, (None,))
    _check(_fn("core", "cpmcu_read_bandwidth")(_p(src), c_long(src.numel() * src.element_size()), _p(out),
                                               c_int(out.shape[0]), _stream()))


class TiledWeight:
    """A weight [N, K] re-laid for the skinny product: [strip of 16 rows][K-block of 128][MFMA i][lane][8],
    lane = 16*g + r holding row 16*strip + r, columns 128*block + 32*i + 8*g .. +8; zero padded."""

    def __init__(self, w: torch.Tensor):
        _need(w, "weight to tile", torch.bfloat16, (None, None))
        N, K = w.shape
        Np, Kp = -(-N // 16) * 16, -(-K // 128) * 128
        if (Np, Kp) != (N, K):
            wp = torch.zeros((Np, Kp), dtype=w.dtype, device=w.device)
            wp[:N, :K] = w
        else:
            wp = w
        self.data = wp.view(Np // 16, 16, Kp // 128, 4, 4, 8).permute(0, 2, 3, 4, 1, 5).contiguous()
        self.N, self.K = N, K

    def first_rows(self, n: int) -> "TiledWeight":
        """The same memory seen as the weight's first n rows (whole strips of 16, or all of it)."""
        if n == self.N:
            return self
        if n <= 0 or n > self.N or n % 16:
            raise KernelError(f"a tiled weight of {self.N} rows gives its first rows in whole strips of 16, not {n}")
        view = object.__new__(TiledWeight)
        view.data, view.N, view.K = self.data[:n // 16], n, self.K
        return view




class QKVRopeWeight:
    """The stacked [q heads; k heads; v heads] x hidden weight re-laid for qkv_rope:
    * the rows of every q and k head as rotation pairs side by side (c, c + hd/2, c + 1, c + 1 + hd/2, ...), v
      heads in their order;
    * cut into runs of R rows, one a workgroup (R from the kernel library: 16, or a few more where that spreads
      the workgroups evenly over the CUs);
    * per run and 128-column block: 16 rows as [MFMA i][lane = 16 g + row][8] (columns 32 i + 8 g ..), then the
      other R - 16 rows as [i][g][row][8]; rows and columns zero padded."""

    def __init__(self, w: torch.Tensor, nh: int, nkv: int, hd: int, rows_per_workgroup: Optional[int] = None):
        total = (nh + 2 * nkv) * hd
        _need(w, "qkv weight", torch.bfloat16, (total, None))
        if hd % 16:
            raise KernelError(f"qkv_rope: head_dim {hd} is no multiple of 16")
        if rows_per_workgroup is None:
            lib = _build.load("qkv")
            lib.cpmcu_qkv_rope_rows_per_workgroup.restype = c_int
            rows_per_workgroup = int(lib.cpmcu_qkv_rope_rows_per_workgroup(c_int(total)))
        R = int(rows_per_workgroup)
        if R < 16 or R > 32 or R % 2:
            raise KernelError(f"qkv_rope: {R} rows a workgroup (an even number from 16 to 32)")
        K = w.shape[1]
        c = torch.arange(hd // 2)
        order = torch.stack([c, c + hd // 2], dim=1).reshape(-1)
        rows = torch.arange(total).view(nh + 2 * nkv, hd).clone()
        rows[:nh + nkv] = rows[:nh + nkv, :1] + order
        n_wg, nkb = -(-total // R), -(-K // 128)
        padded = torch.zeros((n_wg * R, nkb * 128), dtype=w.dtype, device=w.device)
        padded[:total, :K] = w[rows.reshape(-1).to(w.device)]
        blk = padded.view(n_wg, R, nkb, 4, 4, 8)                 # run, row, block, i, g, element
        first = blk[:, :16].permute(0, 2, 3, 4, 1, 5).reshape(n_wg, nkb, 2048)
        rest = blk[:, 16:].permute(0, 2, 3, 4, 1, 5).reshape(n_wg, nkb, 128 * (R - 16))
        self.data = torch.cat([first, rest], dim=2).contiguous()
        self.N, self.K, self.rows_per_workgroup = total, K, R


def qkv_rope_weight(w: torch.Tensor, nh: int, nkv: int, hd: int, rows_per_workgroup: Optional[int] = None
                    ) -> QKVRopeWeight:
    """rows_per_workgroup: None lets the kernel library choose (what the engine does)."""
    return QKVRopeWeight(w, nh, nkv, hd, rows_per_workgroup)


def qkv_rope(x: torch.Tensor, w: QKVRopeWeight, q_out: torch.Tensor, nh: int, nkv: int, hd: int,
             positions: torch.Tensor, tok_slot: torch.Tensor, inv_freq: Optional[torch.Tensor], mscale: float,
             kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
             row_scale: Optional[RowScale] = None, compress: Optional[Tuple[torch.Tensor, int, int]] = None):
    """q, k, v = x . w^T for a step of at most 64 tokens, rotated (inv_freq None: not) and written: q to q_out
    [n, nh*hd], k and v into the paged cache.  w from qkv_rope_weight.  With row_scale, x is the x * w of
    add_norm_columns and the rows of the product are multiplied by the norm's factor before the rotation.
    With compress = (compressed key pool, kernel_size, kernel_stride) the compressed keys that the step's tokens
    complete are written too, as compress_keys would after this call."""
    _need(x, "qkv x", torch.bfloat16, (None, w.K))
    n = x.shape[0]
    if row_scale is not None:
        _need(row_scale.sums, "qkv row sums", torch.float32, (n, None))
    ckpool, ks, st = compress if compress is not None else (None, 0, 0)
    if ckpool is not None:
        # (compressed key pool, kernel_size, kernel_stride): the step's tokens also complete their compressed keys
        if st <= 0 or page_size % st:
            raise KernelError(f"qkv_rope: kernel_stride {st} must divide the cache page of {page_size} tokens")
        _need(ckpool, "qkv compressed key pool", torch.bfloat16, (kpool.shape[0], page_size // st, nkv * hd))
    if not isinstance(w, QKVRopeWeight) or w.N != (nh + 2 * nkv) * hd:
        raise KernelError(f"qkv_rope: the weight must come from qkv_rope_weight for {(nh + 2 * nkv) * hd} rows")
    _need(q_out, "qkv q_out", torch.bfloat16, (n, nh * hd))
    _need(positions, "qkv positions", torch.int32, (n,))
    _need(tok_slot, "qkv token slots", torch.int32, (n,))
    if inv_freq is not None:
        _need(inv_freq, "qkv inv_freq", torch.float32, (hd // 2,))
    _need(kpool, "qkv key pool", torch.bfloat16, (None, page_size, nkv * hd))
    _need(vpool, "qkv value pool", torch.bfloat16, tuple(kpool.shape))
    _need(page_table, "qkv page table", torch.int32, (None, None))
    _check(_fn("qkv", "cpmcu_qkv_rope")(_p(x), c_long(x.stride(0)), _p(w.data), c_int(w.rows_per_workgroup), c_int(n),
                                        c_int(w.K), _p(q_out),
                                        c_int(nh), c_int(nkv), c_int(hd), _p(positions), _p(tok_slot), _p(inv_freq),
                                        c_float(mscale), _p(kpool), _p(vpool), _p(page_table),
                                        c_int(page_table.shape[1]), c_int(page_size),
                                        _p(row_scale.sums if row_scale is not None else None),
                                        c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                        c_float(row_scale.eps if row_scale is not None else 0.0),
                                        _p(ckpool), c_int(ks), c_int(st), _stream()))


def proj_add_norm(a: torch.Tensor, w: "TiledWeight", alpha: float, x: torch.Tensor, weight: torch.Tensor,
                  out: torch.Tensor, sums: torch.Tensor):
    """A branch's last product fused with the residual add and the column part of the norm that follows, for a
    step of at most 64 tokens: x += alpha * (a . w^T) in place (x float32 [n, N], a bfloat16 [n, K], w tiled
    [N, K]); out = bfloat16(x * weight); sums[r, s] = sum of x[r]^2 over the 16 columns of strip s (float32
    [n, ceil(N / 16)]).  As after add_norm_columns, the product that reads `out` applies the row factor."""
    _need(a, "proj a", torch.bfloat16, (None, None))
    n, K = a.shape
    if not isinstance(w, TiledWeight) or w.K != K:
        raise KernelError(f"proj_add_norm: the weight must be tiled for K = {K}")
    N = w.N
    if N % 4 or K % 8:
        raise KernelError(f"proj_add_norm: N={N} must be a multiple of 4 and K={K} of 8")
    _need(x, "proj residual", torch.float32, (n, N))
    _need(weight, "proj norm weight", torch.float32, (N,))
    _need(out, "proj out", torch.bfloat16, (n, N))
    _need(sums, "proj row sums", torch.float32, (n, -(-N // 16)))
    _check(_fn("qkv", "cpmcu_proj_add_norm")(_p(a), c_long(K), _p(w.data), c_int(n), c_int(N), c_int(K),
                                             c_float(alpha), _p(x), _p(weight), _p(out), _p(sums), _stream()))


def gated_strip(x: torch.Tensor, w: "TiledWeight", out: torch.Tensor, row_scale: Optional[RowScale] = None,
                activation="silu"):
    """out = act(x . Wg^T) * (x . Wu^T) (act as in silu_mul) for a step of at most 16 tokens, w tiled with the gate rows first (a
    multiple of 16 of them); out bfloat16 [n, N/2].  With row_scale as in gemm_skinny."""
    _need(x, "gated x", torch.bfloat16, (None, None))
    n, K = x.shape
    if not isinstance(w, TiledWeight) or w.K != K or w.N % 32:
        raise KernelError(f"gated_strip: the weight must be tiled for K = {K} with a multiple of 16 gate rows")
    _need(out, "gated out", torch.bfloat16, (n, w.N // 2))
    if row_scale is not None:
        _need(row_scale.sums, "gated row sums", torch.float32, (n, None))
    _check(_fn("qkv", "cpmcu_gated_strip")(_p(x), c_long(K), _p(w.data), c_int(n), c_int(w.N // 2), c_int(K), _p(out),
                                           _p(row_scale.sums if row_scale is not None else None),
                                           c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                           c_float(row_scale.eps if row_scale is not None else 0.0),
                                           *_act(activation), _stream()))


def gemm_skinny(x: torch.Tensor, w, out: torch.Tensor, alpha: float = 1.0, mode: str = "plain",
                row_scale: Optional[RowScale] = None, activation="silu"):
    """bf16 product for at most 64 rows of x on the matrix cores, streaming w once; w is [N, K] as in the
    checkpoint or a TiledWeight.
    mode 'plain': out [m,N] float32 or bfloat16; 'partial': out float32 [S,m,N], S slices of K to be summed by
    the consumer; 'gated': w holds gate rows then up rows, out bfloat16 [m,N/2] = act(gate) * up (act as in silu_mul).
    With row_scale, x is the x * w of add_norm_columns: the rows of the product are multiplied by the norm's
    factor (before the gate's nonlinearity)."""
    _need(x, "gemm x", torch.bfloat16, (None, None))
    M, K = x.shape
    if row_scale is not None:
        _need(row_scale.sums, "gemm row sums", torch.float32, (M, None))
    tiled = isinstance(w, TiledWeight)
    if tiled:
        if w.K != K:
            raise KernelError(f"gemm weight: tiled for K={w.K}, x has {K} columns")
        N, wt = w.N, w.data
    else:
        _need(w, "gemm weight", torch.bfloat16, (None, K))
        N, wt = w.shape[0], w
    ksplit, omode = 1, 0
    if mode == "plain":
        _need(out, "gemm out", shape=(M, N))
        ldy = N
    elif mode == "partial":
        _need(out, "gemm partial sums", torch.float32, (None, M, N))
        ksplit, omode, ldy = out.shape[0], 1, N
    elif mode == "gated":
        _need(out, "gemm gated out", torch.bfloat16, (M, N // 2))
        omode, ldy = 2, N // 2
    else:
        raise KernelError(f"gemm_skinny: unknown mode '{mode}'")
    _check(_fn("gemm", "cpmcu_gemm_skinny")(_p(x), c_long(K), _p(wt), c_long(K), _p(out), c_long(ldy),
                                            c_int(_code(out)), c_int(omode), c_int(M), c_int(N), c_int(K),
                                            c_int(ksplit), c_float(alpha), c_int(1 if tiled else 0),
                                            _p(row_scale.sums if row_scale is not None else None),
                                            c_int(row_scale.sums.shape[1] if row_scale is not None else 0),
                                            c_float(row_scale.eps if row_scale is not None else 0.0),
                                            *_act(activation), _stream()))


SKINNY_MAX_ROWS = 64


def skinny_ok(x: torch.Tensor, w=None) -> bool:
    return x.dtype == torch.bfloat16 and x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0


def skinny_split(M: int, N: int, K: int) -> int:
    """Slices of K for a skinny product whose consumer sums partial results.  A workgroup streams 64 rows
    of the weight.  Up to 16 rows of x about 1024 small workgroups balance well over the 256 CUs; with more rows
    a workgroup holds 33 or 67 KB of LDS and a CU two or four of them, and a CU with one workgroup more than
    its neighbours ends late: at most one workgroup a CU then (MI355X, 64 rows, us for 2/4/8 slices: q/k/v
    4,608 x 4,096 16.6/19.1/17.7, o 15.7/11.4/13.8, down 51.0/30.5/31.3; 32 rows: 12.5/13.6/13.2, 11.9/9.5/10.6,
    37.8/24.6/25.7).  Every slice should still stream 512 columns, and more rows make the partial sums themselves
    cost traffic."""
    wgs = -(-N // 64)
    cap = 16 if M <= 16 else (8 if M <= 32 else 4)
    most = 5 * compute_units() if M <= 16 else compute_units()
    want = 1
    while want * 2 <= cap and wgs * want * 2 <= most and K // (want * 2) >= 512:
        want *= 2
    if want <= 1:
        return 1
    ks = -(-(-(-K // want)) // 128) * 128
    return -(-K // ks)


# ---------------------------------------------------------------------------
# dispatchers: choose the kernel for a shape and element type
# ---------------------------------------------------------------------------
def library_gemm_ok(x: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Many rows in bf16 with bf16 output: the library's matrix product (the reference calls its vendor's
    library for every linear layer, src/model/linear.cuh:9-37)."""
    return x.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and x.shape[0] > SKINNY_MAX_ROWS


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, alpha: float = 1.0, w_tiled=None):
    """out = alpha * x . w^T with the kernel that suits the element type and the number of rows."""
    M = x.shape[0]
    if w is None and (w_tiled is None or M > SKINNY_MAX_ROWS and out.dtype == torch.bfloat16 and alpha == 1.0):
        raise KernelError(f"linear: {M} rows need the weight in the checkpoint's layout, which this engine let go "
                          f"(it was built for forward passes of at most {SKINNY_MAX_ROWS} tokens)")
    if x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0:
        if M <= SKINNY_MAX_ROWS:
            gemm_skinny(x, w_tiled if w_tiled is not None else w, out, alpha)
            return
        if out.dtype == torch.bfloat16 and alpha == 1.0:
            torch.mm(x, w.t(), out=out)
            return
        # float output for many rows (logits of many positions): the skinny kernel, 64 rows at a time
        for r in range(0, M, SKINNY_MAX_ROWS):
            gemm_skinny(x[r:r + SKINNY_MAX_ROWS], w_tiled if w_tiled is not None else w, out[r:r + SKINNY_MAX_ROWS], alpha)
        return
    gemm_nt_plain(x, w, out, alpha)


def attention(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx,
              sel_blocks=None, sel_count=None, block_size=0, window_blocks=0, head_slopes=None):
    """Attention of the step's queries over the cache, with the kernel that suits the step; writes ``out``.
    head_slopes (float32 [nh], a position encoding's bias of the scores by distance) is taken by the plain
    kernel only, in both element types."""
    if head_slopes is not None:
        attention_plain(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                        sel_blocks, sel_count, block_size, head_slopes)
        return
    if sel_count is None and not ctx.single_token and attention_mfma_ok(q, hd, page_size):
        r, nw = attention_prefill_shape(q.shape[0], nh, nkv, hd)
        tpw = attention_prefill_tokens_per_wave(nh, nkv, r)
        key = ("prefill_tiles", tpw)
        tiles = ctx.extras.get(key)
        if tiles is None:
            tiles = ctx.extras[key] = prefill_tiles(ctx.q_lens, tpw, q.device)
        attention_prefill_mfma(q, out, tiles, nh, nkv, hd, scale, kpool, vpool, page_table, page_size,
                               ctx.positions, ctx.tok_slot, r, nw)
        return
    if attention_mfma_ok(q, hd, page_size, block_size if sel_count is not None else 0):
        n = q.shape[0]
        keys = ctx.max_pos + 1
        if sel_count is not None:
            keys = min(keys, sel_blocks.shape[2] * block_size)
        splits = attention_splits(n, nkv, nh // nkv, keys)
        part_o = part_ml = None
        if splits > 1:
            part_o = ctx.ws.get("attn.part_o", (n, nh, splits, hd), torch.float32)
            part_ml = ctx.ws.get("attn.part_ml", (n, nh, splits, 2), torch.float32)
        attention_mfma(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                       splits, part_o, part_ml, sel_blocks, sel_count, block_size, last_blocks_first=window_blocks)
        return
    attention_plain(q, out, nh, nkv, hd, scale, kpool, vpool, page_table, page_size, ctx.positions, ctx.tok_slot,
                    sel_blocks, sel_count, block_size)


def attention_general_mfma_ok(q: torch.Tensor, hdk: int, hdv: int, page_size: int) -> bool:
    return q.dtype == torch.bfloat16 and hdk % 8 == 0 and hdk <= 1024 and hdv <= 512 and page_size % 32 == 0


def attention_general_splits(n_tokens: int, nkv: int, group: int, pool_hdv: int, max_keys: int) -> int:
    """Shares of a token's keys for attention_general_mfma in steps of few tokens: as attention_splits says (about
    one workgroup a CU, a share of at least 128 keys); four times as many, of at least 64 keys, for values wider
    than 128 features, whose workgroups do not split the keys among their wavefronts and so have less in flight."""
    s = attention_splits(n_tokens, nkv, group, max_keys)
    if pool_hdv > 128 and n_tokens <= compute_units():
        s = max(1, min(s * 4, 64, max_keys // 64))
    return s


def attention_general_mfma(q: torch.Tensor, out: torch.Tensor, nh: int, nkv: int, hdk: int, hdv: int, scale: float,
                           kpool: torch.Tensor, vpool: torch.Tensor, page_table: torch.Tensor, page_size: int,
                           positions: torch.Tensor, tok_slot: torch.Tensor, chunk: int = 0, n_splits: int = 1,
                           part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                           tiles: Optional[torch.Tensor] = None, tokens_per_tile: int = 1, window: int = 0,
                           keep_first: int = 0, sink: Optional[torch.Tensor] = None, v_share: int = 1,
                           gate: Optional[torch.Tensor] = None, softcap: float = 0.0):
    """attention_general in bf16 on the matrix cores (key size a multiple of 8 up to 1024, value size up to 512).
    With n_splits > 1 every token's visible keys are shared among n_splits workgroups and merged afterwards;
    part_o float32 [n, nh, n_splits, hdv] and part_ml float32 [n, nh, n_splits, 2] are its scratch.
    tiles (int32 [T, 2] = first packed token, tokens; prompts of more than 256 tokens with fewer than 16 heads a
    kv head): runs of at most tokens_per_tile consecutive tokens of one sequence,
    which share a matrix-core tile (tokens_per_tile * heads a kv head <= 16).  out is bfloat16, or float32 for a
    consumer that goes on in float (a difference of two maps).  gate (bfloat16 [n, nh*hdv], may be a column slice
    of a wider projection): the output is multiplied element by element with sigmoid(gate) before it is written."""
    _need(q, "attention q", torch.bfloat16, (None, nh * hdk))
    n = q.shape[0]
    if out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"attention out: dtype {out.dtype} (bfloat16 or float32)")
    _need(out, "attention out", out.dtype, (n, nh * hdv))
    _need(kpool, "attention key pool", torch.bfloat16, (None, page_size, None))
    _need(vpool, "attention value pool", torch.bfloat16, (kpool.shape[0], page_size, None))
    nvh = _value_heads(nkv, v_share)
    if kpool.shape[2] % nkv or vpool.shape[2] % nvh:
        raise KernelError(f"attention_general: pools of {kpool.shape[2]} / {vpool.shape[2]} features do not hold {nkv} / {nvh} heads")
    _need(page_table, "attention page table", torch.int32, (None, None))
    _need(positions, "attention positions", torch.int32, (n,))
    _need(tok_slot, "attention token slots", torch.int32, (n,))
    if n_splits > 1:
        _need(part_o, "attention partial outputs", torch.float32, (n, nh, n_splits, hdv))
        _need(part_ml, "attention partial max/sum", torch.float32, (n, nh, n_splits, 2))
    if tiles is not None:
        _need(tiles, "attention tiles", torch.int32, (None, 2))
    if sink is not None:
        _need(sink, "attention sink", torch.float32, (nh,))
    ld_gate = 0
    if gate is not None:
        ld_gate = _ld(gate, "attention gate")
        if gate.dtype != torch.bfloat16 or tuple(gate.shape) != (n, nh * hdv):
            raise KernelError(f"attention gate: {gate.dtype} {tuple(gate.shape)}, expected bfloat16 {(n, nh * hdv)}")
    _check(_fn("attention_general", "cpmcu_attention_general_mfma")(
        _p(q), _p(out), c_int(1 if out.dtype == torch.float32 else 0), _p(part_o), _p(part_ml), c_int(n), c_int(nh),
        c_int(nkv), c_int(hdk), c_int(hdv),
        c_int(kpool.shape[2] // nkv), c_int(vpool.shape[2] // nvh), c_float(scale), c_int(chunk), c_int(window),
        c_int(keep_first), _p(sink), _p(kpool), _p(vpool),
        _p(page_table), c_int(page_table.shape[1]), c_int(page_size), _p(positions), _p(tok_slot), c_int(n_splits),
        _p(tiles), c_int(tiles.shape[0] if tiles is not None else 0), c_int(tokens_per_tile), c_int(v_share),
        _p(gate), c_long(ld_gate), c_float(softcap or 0.0), _stream()))


def attention_general_tokens_per_tile(n_tokens: int, nh: int, nkv: int, pool_hdv: int) -> int:
    """Tokens that share a matrix-core tile in attention_general_mfma: prompts of more than 256 tokens whose
    kv heads serve fewer than 16 query heads fill the tile's 16 columns with the heads of several consecutive
    tokens; 1 everywhere else."""
    group = nh // nkv
    if n_tokens <= 256 or group > 8:
        return 1
    return 16 // group


def reserve_attention_general(ws, dtype, nh: int, nkv: int, hdv: int, pool_hdv: int, max_keys: int, max_step_tokens: int):
    """Ask the workspace for the shares of attention_any's split steps at their largest (they grow with the
    context), so that no later step has to."""
    if dtype != torch.bfloat16:
        return
    most = max((n * attention_general_splits(n, nkv, nh // nkv, pool_hdv, max_keys)
                for n in range(1, min(max_step_tokens, compute_units()) + 1)), default=0)
    if most > 1:
        ws.get("attn.gpart_o", (most, nh, hdv), torch.float32)
        ws.get("attn.gpart_ml", (most, nh, 2), torch.float32)


def attention_any(q, out, nh, nkv, hdk, hdv, scale, kpool, vpool, page_table, page_size, ctx, chunk: int = 0,
                  window: int = 0, keep_first: int = 0, sink: Optional[torch.Tensor] = None, v_share: int = 1,
                  gate: Optional[torch.Tensor] = None, softcap: float = 0.0) -> bool:
    """Attention with key and value sizes of their own and an optional mask (chunks, or a sliding window with kept
    first tokens) and softmax sink, with the kernel that suits the step; writes ``out`` [n, nh*hdv] (q's type, or
    float32).  v_share: runs of that many neighbouring key heads read one value head.  gate [n, nh*hdv]: an output
    gate that the matrix-core kernel applies as it writes (out * sigmoid(gate)); returns whether it did, so that
    the caller applies it itself after the other kernels.  softcap c > 0: scaled scores pass c tanh(s / c)."""
    pool_hdv = vpool.shape[2] // _value_heads(nkv, v_share)
    if (hdk == hdv and chunk == 0 and window == 0 and sink is None and hdk <= 256 and hdk % 16 == 0
            and kpool.shape[2] == nkv * hdk and v_share == 1 and not softcap):
        attention(q, out, nh, nkv, hdk, scale, kpool, vpool, page_table, page_size, ctx)
        return False
    if attention_general_mfma_ok(q, hdk, hdv, page_size):
        n = q.shape[0]
        keys = ctx.max_pos + 1
        if chunk:
            keys = min(keys, chunk)
        if window:
            keys = min(keys, window + keep_first)
        splits = attention_general_splits(n, nkv, nh // nkv, pool_hdv, keys) if ctx.single_token else 1
        part_o = part_ml = None
        if splits > 1:
            part_o = ctx.ws.get("attn.gpart_o", (n, nh, splits, hdv), torch.float32)
            part_ml = ctx.ws.get("attn.gpart_ml", (n, nh, splits, 2), torch.float32)
        tiles, tpt = None, 1
        if not ctx.single_token:
            tpt = attention_general_tokens_per_tile(n, nh, nkv, pool_hdv)
            if tpt > 1:
                key = ("prefill_tiles", tpt)
                tiles = ctx.extras.get(key)
                if tiles is None:
                    tiles = ctx.extras[key] = prefill_tiles(ctx.q_lens, tpt, q.device)
        attention_general_mfma(q, out, nh, nkv, hdk, hdv, scale, kpool, vpool, page_table, page_size, ctx.positions,
                               ctx.tok_slot, chunk, splits, part_o, part_ml, tiles, tpt, window, keep_first, sink, v_share,
                               gate, softcap)
        return gate is not None
    if out.dtype != q.dtype:
        # the plain kernel writes the type it reads: through scratch of that type
        tmp = ctx.ws.get("attn.gout_plain", tuple(out.shape), q.dtype)
        attention_general(q, tmp, nh, nkv, hdk, hdv, scale, kpool, vpool, page_table, page_size, ctx.positions,
                          ctx.tok_slot, chunk, window, keep_first, sink, v_share, softcap)
        out.copy_(tmp)
        return False
    attention_general(q, out, nh, nkv, hdk, hdv, scale, kpool, vpool, page_table, page_size, ctx.positions,
                      ctx.tok_slot, chunk, window, keep_first, sink, v_share, softcap)
    return False
