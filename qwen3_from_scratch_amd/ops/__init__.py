"""The operations the model is made of, each a hand-written HIP kernel.

Every function checks its operands on the host (device, dtype, contiguity and
the shapes the kernel's grid assumes) and then launches on the current HIP
stream. Tensors must live on the GPU: there is no host implementation, and a
missing or unbuildable extension raises `ExtensionError`.

Activations and matrices are bfloat16 or float32 (the same for all operands of
one call unless stated); the residual stream, rotation tables, softmax
statistics and logits are float32 in both modes.
"""

import ctypes
import json
import os

import torch

from .build import ExtensionError, build_all, library, loaded_libraries

__all__ = [
    "ExtensionError",
    "build_all",
    "loaded_libraries",
    "embed_rows",
    "rmsnorm",
    "rmsnorm_addend",
    "rope_table",
    "qk_norm_rope_store",
    "paged_attention",
    "decode_attention",
    "decode_attention_takes",
    "swiglu",
    "gated_act",
    "layernorm_addend",
    "moe_glu_experts",
    "glu_clamped",
    "gelu",
    "latent_prepare",
    "headwise_linear",
    "rotate_heads",
    "latent_attention",
    "moe_route",
    "moe_experts",
    "moe_gated_experts",
    "embed_streams",
    "hyper_norm",
    "causal_conv",
    "mamba2_scan",
    "gated_rmsnorm",
    "block_gates",
    "rglru_scan",
    "retention_scan",
    "softcap_prepare",
    "headnorm_prepare",
    "channel_delta",
    "softcap_attention",
    "scaled_sum",
    "linear",
    "linear_plain",
    "linear_swiglu",
    "linear_residual_norm",
    "matmul_candidates",
    "matmul_kernels",
    "matmul_init",
    "matmul_table",
    "matmul_tuner",
    "matmul_rows_key",
    "matmul_fused_plan",
    "gemm_tiles",
    "gemm_tiles_configs",
    "gemm_tiles_splits",
    "matmul_plan",
    "stream_plan",
    "tile_weight",
    "sample",
    "measured_read_rate",
    "measured_matrix_rate",
]

_DT = {torch.float32: 0, torch.bfloat16: 1}
_UNSUPPORTED = 10002          # a launcher's refusal of a size it has no kernel for
_DECLINED = 1                 # the fused product of 17 to 128 rows did nothing: the plain product is faster here


class OperandError(ValueError):
    """An operand has a shape, dtype or placement the kernel does not take."""


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle without a Stream object around it


def _stream():
    """The current device's current stream, as the launchers take it. Every operation asks, some
    hundreds of times in a step that is not a graph replay, so the short way is taken where this
    PyTorch has it (a fifth of such a step's host time otherwise)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond, message):
    if not cond:
        raise OperandError(message)


def _dev(*tensors):
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "operands must be on the GPU; there is no host implementation")
        _need(t.is_contiguous(), "operands must be contiguous")


def _check(status, what):
    if status >= 20000:
        raise RuntimeError("%s failed: hipBLASLt status %d" % (what, status - 20000))
    if status != 0:
        raise RuntimeError("%s failed: HIP error %d" % (what, status))


_KINDS = {"plain": 0, "scaled": 1, "scaled_swiglu": 2, "residual": 3}
TABLE_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "matmul_table.json")
_table_loaded = False


def _matmul():
    """The many-row product library, with the table of kernel choices loaded at its first use."""
    global _table_loaded
    lib = library("matmul")
    if not _table_loaded:
        _table_loaded = True
        if os.path.isfile(TABLE_FILE):
            with open(TABLE_FILE, encoding="utf-8") as fh:
                _add_to_table(lib, json.load(fh)["entries"])
    return lib


def _add_to_table(lib, entries):
    for e in entries:
        out = _DT[getattr(torch, e.get("out", "bfloat16"))]
        _check(lib.q3_matmul_table_add(_KINDS[e["kind"]], int(e["rows"]), int(e["N"]), int(e["K"]), out,
                                       int(e.get("library", 0)), int(e.get("own", -1)), int(e.get("splits", 1))),
               "matmul_table")


def matmul_init():
    """Allocate the many-row products' workspace and buffers on the current device now (a model
    being built calls this), so that no product inside a step allocates."""
    _check(_matmul().q3_matmul_init(), "matmul_init")


def matmul_table(entries, clear=False):
    """Load kernel choices: each entry {"kind": "plain" | "scaled" | "scaled_swiglu" | "residual",
    "rows": rounded rows (`matmul_rows_key`), "N", "K", "out": "bfloat16" | "float32",
    "library": the library's candidate number, or "own": tile shape and "splits": shares of K}.
    Sizes without an entry follow the rules of thumb. Sizes already met keep their kernel."""
    lib = _matmul()                      # the package's own table first, if it is not in yet
    if clear:
        _check(lib.q3_matmul_table_clear(), "matmul_table")
    _add_to_table(lib, entries)


def matmul_rows_key(kind, M):
    """The rows a table entry for `M` rows is filed under (sizes within a step of rows share one)."""
    return int(library("matmul").q3_matmul_rows_key(_KINDS[kind], int(M)))


def matmul_tuner(on):
    """With the tuner on, a product size first met outside a graph capture has its candidate
    kernels timed on the caller's operands and keeps the fastest for the life of the process
    (`matmul_plan`, `matmul_fused_plan` tell which): the way the table is made. Off (the
    default), kernels are chosen by the table and the rules alone, the same in every process."""
    _check(_matmul().q3_matmul_set_mode(1 if on else 0), "matmul_tuner")


def matmul_candidates(n):
    """How many of the vendor library's candidate kernels the tuner times for a new size."""
    _check(_matmul().q3_matmul_set_candidates(int(n)), "matmul_candidates")


def matmul_kernels(which):
    """Which kernels a product with many rows may go to: "both" (the table and the rules decide
    between the vendor library and the hand-written tiled kernel; the default), "library" (the
    library's first candidate), or "own" (the hand-written kernel wherever it takes the size: an
    inner size that is a multiple of 64). A change makes every size choose anew."""
    modes = {"both": 0, "library": 1, "own": 2}
    _need(which in modes, "which is one of %s" % ", ".join(sorted(modes)))
    _check(_matmul().q3_matmul_set_kernels(modes[which]), "matmul_kernels")


def matmul_plan(M, N, K, out_dtype=torch.bfloat16):
    """What serves a plain product of this size on the current device, or None if it has not
    been met: (candidates timed (1 without the tuner), index chosen, microseconds of the first
    candidate, of the chosen one, the hand-written kernel's tile shape if that serves it, else
    -1, over how many blocks it shares K out, the library's candidate number)."""
    info = (ctypes.c_float * 7)()
    if not _matmul().q3_matmul_plan(int(M), int(N), int(K), _DT[out_dtype], info):
        return None
    return int(info[0]), int(info[1]), float(info[2]), float(info[3]), int(info[4]), int(info[5]), int(info[6])


def matmul_fused_plan(kind, M, N, K):
    """What serves a product of 17 to 128 rows that carries a norm (`kind` "scaled",
    "scaled_swiglu" or "residual"): (tile shape or -1 for the library's product with the norm's
    work behind it, shares of K); None with the tuner on for a size it has not met."""
    info = (ctypes.c_int * 2)()
    if not _matmul().q3_matmul_fused_plan(_KINDS[kind], int(M), int(N), int(K), info):
        return None
    return int(info[0]), int(info[1])


def gemm_tiles_configs():
    """How many tile shapes the hand-written tiled product offers."""
    return int(library("matmul").q3_gemm_tiles_configs())


def gemm_tiles_splits(config, M, N, K):
    """Over how many blocks per tile the tiled product would share K out so that the chip is
    filled once (1: its tiles alone do)."""
    return int(library("matmul").q3_gemm_tiles_splits(int(config), int(M), int(N), int(K)))


def gemm_tiles(x, weight, config=0, out_dtype=None, swiglu=False, out=None, splits=1):
    """The hand-written tiled matrix-core product alone, with tile shape `config`: x (M, K) and
    weight (N, K) bfloat16, K a multiple of 64; out (M, N) bfloat16 or float32, or with `swiglu`
    (weight rows interleave gate and up) out (M, N / 2) bfloat16 = silu(gate) * up. With
    `splits` > 1 (N a multiple of 4) K is shared out over that many blocks per tile and their
    float32 partial products are added by a second kernel, which then also applies the activation."""
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "x and weight must be bfloat16")
    M, K = x.shape
    N = weight.shape[0]
    _need(M > 0 and K >= 64 and K % 64 == 0, "the inner size must be a multiple of 64")
    _need(0 <= config < gemm_tiles_configs(), "no such tile shape")
    out_dtype = out_dtype or torch.bfloat16
    _need(out_dtype in _DT and not (swiglu and (out_dtype != torch.bfloat16 or N % 2)),
          "out is bfloat16 or float32; with swiglu bfloat16 and an even number of weight rows")
    _need(1 <= splits <= min(64, K // 64) and (splits == 1 or N % 4 == 0),
          "K is shared out over 1 to min(64, K / 64) blocks, and then N is a multiple of 4")
    shape = (M, N // 2) if swiglu else (M, N)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out.shape == shape and out.dtype == out_dtype, "out must be %s of out_dtype" % (shape,))
    partials = torch.empty((splits * M * N,), dtype=torch.float32, device=x.device) if splits > 1 else None
    _check(library("matmul").q3_gemm_tiles(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[out_dtype],
                                           1 if swiglu else 0, int(config), int(splits), _ptr(partials), _stream()),
           "gemm_tiles")
    return out


def embed_rows(ids, table, out=None, scale=1.0):
    """out[t, :] = float32(table[ids[t], :]) * scale. ids int32 (T,), table (V, H)."""
    _dev(ids, table, out)
    _need(ids.dtype == torch.int32 and ids.dim() == 1, "ids must be int32 (T,)")
    _need(table.dim() == 2 and table.dtype in _DT, "table must be (V, H) bfloat16 or float32")
    T, (V, H) = ids.shape[0], table.shape
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.shape == (T, H) and out.dtype == torch.float32, "out must be float32 (T, H)")
    if T:
        _check(library("elementwise").q3_embed_rows(
            _ptr(ids), _ptr(table), _ptr(out), T, H, V, ctypes.c_float(scale), _DT[table.dtype], _stream()), "embed_rows")
    return out


GATE_KINDS = {"silu": 0, "gelu_tanh": 1, "gelu_erf": 2}


def gated_act(gate_up, kind="silu", out=None):
    """out[:, j] = act(gate_up[:, 2j]) * gate_up[:, 2j + 1]: gate and up interleaved, (T, 2I) -> (T, I).
    `kind`: "silu" for g / (1 + exp(-g)), "gelu_tanh" for 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))),
    "gelu_erf" for 0.5 g (1 + erf(g / sqrt 2)); float32 arithmetic, rounded once."""
    _dev(gate_up, out)
    _need(kind in GATE_KINDS, "kind is one of %s" % ", ".join(sorted(GATE_KINDS)))
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0 and gate_up.dtype in _DT,
          "gate_up must be (T, 2I) bfloat16 or float32")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.shape == (T, I) and out.dtype == gate_up.dtype, "out must be (T, I) of the input's dtype")
    if T:
        _check(library("elementwise").q3_gated_act(
            _ptr(gate_up), _ptr(out), T, I, GATE_KINDS[kind], _DT[gate_up.dtype], _stream()), "gated_act")
    return out


def swiglu(gate_up, out=None):
    """out[:, j] = silu(gate_up[:, 2j]) * gate_up[:, 2j + 1]: gate and up interleaved, (T, 2I) -> (T, I)."""
    return gated_act(gate_up, "silu", out=out)


def glu_clamped(gate_up, limit, slope, bias=None, scale=None, scale_index=None, out_dtype=None):
    """A gated unit with clamped branches over rows that interleave the two (column 2j the gate's,
    2j + 1 the other branch's): a = gate_up * w + bias; g = min(a_gate, limit), u = clamp(a_up, -limit,
    limit); out[t, j] = g * sigmoid(slope * g) * (u + 1), float32 throughout, rounded once. `bias` float32
    (2I,) over the interleaved columns; `scale` float32 (n,) with w = scale[scale_index[t]] (`scale_index`
    int32 (T,)) or scale[t]: a number per row that multiplied the product's input. gate_up (T, 2I);
    the result has `out_dtype` (gate_up's by default)."""
    _dev(gate_up, bias, scale, scale_index)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0 and gate_up.dtype in _DT and gate_up.is_contiguous(),
          "gate_up must be (T, 2I), contiguous, bfloat16 or float32")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if bias is not None:
        _f32(bias, (2 * I,), "bias")
    if scale is not None:
        _need(scale.dtype == torch.float32 and scale.dim() == 1 and scale.is_contiguous(), "scale must be float32 (n,)")
        if scale_index is not None:
            _need(scale_index.dtype == torch.int32 and scale_index.shape == (T,), "scale_index must be int32 (T,)")
        else:
            _need(scale.shape == (T,), "a scale without an index has one number per row")
    else:
        _need(scale_index is None, "an index needs a scale")
    _need(limit > 0, "limit must be positive")
    out_dtype = out_dtype or gate_up.dtype
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    out = torch.empty((T, I), dtype=out_dtype, device=gate_up.device)
    if T and I:
        _check(library("elementwise").q3_glu_clamped(
            _ptr(gate_up), _ptr(bias), _ptr(scale), _ptr(scale_index), _ptr(out), T, I, ctypes.c_float(limit),
            ctypes.c_float(slope), _DT[gate_up.dtype], _DT[out_dtype], _stream()), "glu_clamped")
    return out


def rmsnorm(x, weight, eps, out_dtype, delta=None, rows=None, write_back=True, out=None):
    """Root-mean-square norm of the float32 residual stream.

    For each output row r (source row s = rows[r], or r when rows is None):
    v = x[s] + delta[s] (delta optional), written back to x[s] if `write_back`
    and delta is given; out[r] = v * rsqrt(mean(v^2) + eps) * weight, rounded
    once to `out_dtype`. All arithmetic is float32.
    """
    _dev(x, weight, delta, rows, out)
    _need(x.dim() == 2 and x.dtype == torch.float32, "x must be float32 (T, H)")
    T, H = x.shape
    _need(weight.shape == (H,) and weight.dtype in _DT, "weight must be (H,) bfloat16 or float32")
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    if delta is not None:
        _need(delta.shape == (T, H) and delta.dtype == out_dtype,
              "delta must be (T, H) of the activation dtype")
    n_out = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1, "rows must be int32 (R,)")
        n_out = rows.shape[0]
    if out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=x.device)
    _need(out.shape == (n_out, H) and out.dtype == out_dtype, "out must be (rows, H) of out_dtype")
    if n_out:
        _check(library("norm").q3_rmsnorm(
            _ptr(x), _ptr(delta), _ptr(weight), _ptr(rows), _ptr(out), n_out, T, H,
            ctypes.c_float(eps), _DT[out_dtype], _DT[weight.dtype],
            1 if (write_back and delta is not None) else 0, _stream()), "rmsnorm")
    return out


def rmsnorm_addend(x, weight, eps, out_dtype, delta=None, delta_weight=None, delta_eps=0.0, bias=None, rows=None,
                   write_back=True, out=None, delta_bias=None, plain=False):
    """The norm of the float32 stream behind an addend that is itself normalised first, and behind
    a vector added to every row, all in float32 and in one kernel:

    a = (delta[s] + delta_bias) * rsqrt(mean(.^2) + delta_eps) * delta_weight (or delta[s] + delta_bias
    as it is without `delta_weight`, or nothing); v = x[s] + a + bias; x[s] = v if `write_back`;
    out[r] = v * rsqrt(mean(v^2) + eps) * weight, rounded once to `out_dtype`. With `weight` None
    only the stream is brought up to date and None is returned, unless `plain` asks for the stream
    itself: out[r] = v, rounded once (what a sublayer reads that has no norm before it). `delta`
    (T, H) has the activation dtype, `bias` and `delta_bias` (H,) are float32, `rows` as in `rmsnorm`."""
    _dev(x, weight, delta, delta_weight, bias, rows, out, delta_bias)
    _need(x.dim() == 2 and x.dtype == torch.float32, "x must be float32 (T, H)")
    T, H = x.shape
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    w_dtype = None
    for w in (weight, delta_weight):
        if w is not None:
            _need(w.shape == (H,) and w.dtype in _DT and w_dtype in (None, w.dtype), "norm weights must be (H,) of one dtype")
            w_dtype = w.dtype
    if delta is not None:
        _need(delta.shape == (T, H) and delta.dtype == out_dtype, "delta must be (T, H) of the activation dtype")
    _need(delta is not None or (delta_weight is None and delta_bias is None), "a delta weight or bias needs a delta")
    for b in (bias, delta_bias):
        if b is not None:
            _need(b.shape == (H,) and b.dtype == torch.float32, "a bias must be float32 (H,)")
    _need(not plain or weight is None, "the plain stream is read without a weight")
    n_out = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1, "rows must be int32 (R,)")
        n_out = rows.shape[0]
    if weight is None and not plain:
        _need(out is None and rows is None, "without a weight there is no output")
    elif out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=x.device)
    if out is not None:
        _need(out.shape == (n_out, H) and out.dtype == out_dtype, "out must be (rows, H) of out_dtype")
    write = 1 if (write_back and rows is None and (delta is not None or bias is not None)) else 0
    if n_out:
        _check(library("norm").q3_rmsnorm_addend(
            _ptr(x), _ptr(delta), _ptr(delta_weight), ctypes.c_float(delta_eps), _ptr(delta_bias), _ptr(bias), _ptr(weight),
            _ptr(rows), _ptr(out), n_out, T, H, ctypes.c_float(eps), _DT[out_dtype], _DT[w_dtype or torch.float32], write,
            _stream()), "rmsnorm_addend")
    return out


def layernorm_addend(x, weight, bias, eps, out_dtype, delta=None, extra=None, vec=None, rows=None, write_back=True):
    """A layer norm with a weight and a bias of the float32 stream behind everything the stream still
    lacks, in float32 and in one kernel. For each output row r (source row s = rows[r], or r):

    v = x[s] + delta[s] + extra[s] + vec, every addend optional: `delta` (T, H) in the activation dtype (a
    part's result), `extra` float32 (T, H) (rows that join as they are), `vec` float32 (H,) (one vector for
    every row); x[s] = v if `write_back` and `rows` is None; out[r] = (v - mean(v)) * rsqrt(mean((v -
    mean(v))^2) + eps) * weight + bias, rounded once to `out_dtype`. `weight` and `bias` are float32 (H,)
    (`bias` None: none). With `weight` None only the stream is brought up to date and None is returned."""
    _dev(x, weight, bias, delta, extra, vec, rows)
    _need(x.dim() == 2 and x.dtype == torch.float32, "x must be float32 (T, H)")
    T, H = x.shape
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    for w, what in ((weight, "weight"), (bias, "bias"), (vec, "vec")):
        if w is not None:
            _f32(w, (H,), what)
    _need(weight is not None or bias is None, "a bias comes with a weight")
    if delta is not None:
        _need(delta.shape == (T, H) and delta.dtype == out_dtype, "delta must be (T, H) of the activation dtype")
    if extra is not None:
        _f32(extra, (T, H), "extra")
    n_out = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1, "rows must be int32 (R,)")
        n_out = rows.shape[0]
    _need(weight is not None or rows is None, "without a weight there is no output")
    out = torch.empty((n_out, H), dtype=out_dtype, device=x.device) if weight is not None else None
    write = 1 if (write_back and rows is None and (delta is not None or extra is not None or vec is not None)) else 0
    if n_out and (out is not None or write):
        _check(library("norm").q3_layernorm_addend(
            _ptr(x), _ptr(delta), _ptr(extra), _ptr(vec), _ptr(weight), _ptr(bias), _ptr(rows), _ptr(out), n_out, T, H,
            ctypes.c_float(eps), _DT[out_dtype], write, _stream()), "layernorm_addend")
    return out


def gelu(x, kind="erf", out=None):
    """gelu(x) elementwise in float32, rounded once. `kind`: "erf" for 0.5 z (1 + erf(z / sqrt 2)),
    "tanh" for 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""
    _dev(x, out)
    _need(x.dtype in _DT and kind in GELU_KINDS, "x bfloat16 or float32; kind erf or tanh")
    if out is None:
        out = torch.empty_like(x)
    _need(out.shape == x.shape and out.dtype == x.dtype, "out must be like x")
    if x.numel():
        _check(library("elementwise").q3_gelu(_ptr(x), _ptr(out), ctypes.c_long(x.numel()), GELU_KINDS[kind],
                                              _DT[x.dtype], _stream()), "gelu")
    return out


GELU_KINDS = {"erf": 0, "tanh": 1}


def latent_prepare(down, q_rank, kv_rank, rot_dim, q_weight, kv_weight, eps, inv_freq, rot_factor, positions, seq_index,
                   block_table=None, cache=None):
    """The narrow vectors of latent attention from their joint down-projection, in float32:

    down (T, n), n >= q_rank + kv_rank + rot_dim, rows possibly apart, holds [query latent | key/value
    latent | key part to be rotated | ...]; rot_dim may be 0 (keys without a rotated part; `inv_freq`
    None). Returns the normalised query latent (T, q_rank) (`q_weight`, `eps`), and writes
    [normalised key/value latent (`kv_weight`) | rotated key part] as the token's row of `cache`
    (pages, page, kv_rank + rot_dim) at page block_table[seq_index[t], position // page]; entries
    below zero are skipped, nothing is written without a cache. The rotation turns the pairs
    (2i, 2i + 1), i < len(inv_freq), by float32(position) * inv_freq[i], with cos and sin
    multiplied by `rot_factor`; what lies beyond the pairs passes."""
    _dev(q_weight, kv_weight, inv_freq, positions, seq_index, block_table, cache)
    R = q_rank + kv_rank + rot_dim
    _need(down.is_cuda and down.dim() == 2 and down.shape[1] >= R and down.dtype in _DT and down.stride(1) == 1,
          "down must be (T, q_rank + kv_rank + rot_dim or more) with its columns side by side")
    T = down.shape[0]
    _need(q_weight.shape == (q_rank,) and kv_weight.shape == (kv_rank,) and q_weight.dtype in _DT
          and kv_weight.dtype == q_weight.dtype, "norm weights (q_rank,) and (kv_rank,) of one dtype")
    pairs = 0
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 2 * inv_freq.shape[0] <= rot_dim,
              "inv_freq float32, at most rot_dim / 2 pairs")
        pairs = inv_freq.shape[0]
    for t in (positions, seq_index):
        _need(t.dtype == torch.int32 and t.shape == (T,), "positions and seq_index must be int32 (T,)")
    page = pages = stride = rows = 0
    if cache is not None:
        _need(block_table is not None and block_table.dim() == 2 and block_table.dtype == torch.int32,
              "a cache needs an int32 block table (B, W)")
        _need(cache.dim() == 3 and cache.shape[2] == kv_rank + rot_dim and cache.dtype == down.dtype,
              "cache must be (pages, page, kv_rank + rot_dim) of the activation dtype")
        pages, page = cache.shape[0], cache.shape[1]
        rows, stride = block_table.shape
    cq = torch.empty((T, q_rank), dtype=down.dtype, device=down.device)
    if T:
        _check(library("latent").q3_latent_prepare(
            _ptr(down), ctypes.c_long(down.stride(0)), T, q_rank, kv_rank, rot_dim, _ptr(q_weight), _ptr(kv_weight),
            _DT[q_weight.dtype], ctypes.c_float(eps), _ptr(inv_freq), pairs, ctypes.c_float(rot_factor), _ptr(positions),
            _ptr(seq_index), _ptr(block_table), stride, rows, _ptr(cache), page, pages, _ptr(cq), _DT[down.dtype],
            _stream()), "latent_prepare")
    return cq


def headwise_linear(x, weight, out=None):
    """out[t, h, :] = weight[h] x[t, h, :]: x (T, H, I) seen through strides (its last axis
    contiguous), weight (H, O, I) contiguous, out (T, H, O) likewise seen through strides; float32
    sums. bfloat16 with I in steps of 32 and rows of x that start at multiples of 16 bytes runs on
    the matrix cores, everything else as float32 multiply-adds in the order of I."""
    _dev(weight)
    _need(x.is_cuda and x.dim() == 3 and x.stride(2) == 1 and weight.dim() == 3 and x.dtype in _DT
          and weight.dtype == x.dtype, "x (T, H, I) with a contiguous last axis, weight (H, O, I), one dtype")
    T, H, I = x.shape
    O = weight.shape[1]
    _need(weight.shape == (H, O, I), "weight must be (H, O, I)")
    if out is None:
        out = torch.empty((T, H, O), dtype=x.dtype, device=x.device)
    _need(out.is_cuda and out.shape == (T, H, O) and out.stride(2) == 1 and out.dtype == x.dtype, "out must be (T, H, O)")
    cores = (x.dtype == torch.bfloat16 and I % 32 == 0 and x.stride(0) % 8 == 0 and x.stride(1) % 8 == 0
             and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)
    if T:
        _check(library("latent").q3_headwise_linear(
            _ptr(x), ctypes.c_long(x.stride(0)), x.stride(1), _ptr(weight), _ptr(out), ctypes.c_long(out.stride(0)),
            out.stride(1), T, H, I, O, _DT[x.dtype], 1 if cores else 0, _stream()), "headwise_linear")
    return out


def rotate_heads(x, out, inv_freq, rot_factor, positions):
    """out[t, h, :] = x[t, h, :] with its pairs (2i, 2i + 1), i < len(inv_freq), turned by
    float32(positions[t]) * inv_freq[i] (cos and sin times `rot_factor`), the rest copied; x and
    out (T, H, n) seen through strides."""
    _dev(inv_freq, positions)
    _need(x.is_cuda and out.is_cuda and x.dim() == 3 and out.shape == x.shape and x.stride(2) == 1
          and out.stride(2) == 1 and x.dtype in _DT and out.dtype == x.dtype, "x and out (T, H, n) of one dtype")
    T, H, n = x.shape
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and 2 * inv_freq.shape[0] <= n, "inv_freq float32")
    _need(positions.dtype == torch.int32 and positions.shape == (T,), "positions int32 (T,)")
    if T:
        _check(library("latent").q3_rotate_heads(
            _ptr(x), ctypes.c_long(x.stride(0)), x.stride(1), _ptr(out), ctypes.c_long(out.stride(0)), out.stride(1),
            T, H, n, inv_freq.shape[0], _ptr(inv_freq), ctypes.c_float(rot_factor), _ptr(positions), _DT[x.dtype],
            _stream()), "rotate_heads")
    return out


def latent_attention(q, cache, value_dim, block_table, cu_seqlens_q, kv_lens, max_q_len, scale, window=0,
                     general=False, max_kv_len=0, sink=None, gate=None):
    """Causal softmax attention of every head's query rows over one shared sequence of cached rows.

    q (T, H, Dk) contiguous; cache (pages, page, Dk): the row of sequence b's position j lies in
    page block_table[b, j // page]; a row is the key in full and the value in its first
    `value_dim` numbers. The query of token i of sequence b (position kv_lens[b] - q_len + i) sees
    positions j <= its own and, with window > 0, only those fewer than `window` behind it.
    Returns (T, H, value_dim). Float32 scores, statistics and sums. bfloat16 with Dk in steps of 32
    (up to 576) and value_dim in steps of 16 (up to 512) runs on the matrix cores; everything
    else, and everything with `general=True`, takes the kernel of float32 multiply-adds.
    `max_q_len` bounds the sequences' rows and `max_kv_len` (0: unknown) their keys: a step of few
    rows over many keys shares the keys out over several blocks per row tile. `sink` float32 (H,):
    head h's softmax has exp(sink[h]) as one more term of its denominator, which has no key and no value
    and is not scaled. `gate` (T, H) of q's dtype, rows possibly apart: head h's result is multiplied by
    sigmoid(gate[t, h])."""
    _dev(q, cache, block_table, cu_seqlens_q, kv_lens, sink)
    _need(q.dim() == 3 and q.dtype in _DT and cache.dim() == 3 and cache.dtype == q.dtype
          and cache.shape[2] == q.shape[2], "q (T, H, Dk) and cache (pages, page, Dk) of one dtype")
    T, H, Dk = q.shape
    B = kv_lens.shape[0]
    _need(0 < value_dim <= Dk, "the value is a leading part of the cached row")
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.shape == (B + 1,) and kv_lens.dtype == torch.int32,
          "cu_seqlens_q int32 (B + 1,), kv_lens int32 (B,)")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.shape[0] >= B,
          "block_table must be int32 (B, W)")
    gate_stride = 0
    if sink is not None:
        _f32(sink, (H,), "sink")
    if gate is not None:
        gate_stride = _rows_view(gate, "gate")
        _need(gate.shape == (T, H) and gate.dtype == q.dtype, "gate must be (T, H) of q's dtype")
    out = torch.empty((T, H, value_dim), dtype=q.dtype, device=q.device)
    if T and B:
        lib = library("latent")
        splits, partial = 1, None
        if not general and lib.q3_latent_attention_fast_path(Dk, value_dim, _DT[q.dtype]):
            splits = _latent_splits(T, B, H, max_q_len, max_kv_len, window)
            if splits > 1:
                partial = torch.empty((T * H * splits * (value_dim + 2),), dtype=torch.float32, device=q.device)
        _check(lib.q3_latent_attention(
            _ptr(q), _ptr(out), _ptr(cache), cache.shape[0], _ptr(block_table), block_table.shape[1],
            _ptr(cu_seqlens_q), _ptr(kv_lens), B, T, H, Dk, value_dim, cache.shape[1], ctypes.c_float(scale), int(window),
            int(max_q_len), _DT[q.dtype], 1 if general else 0, splits, _ptr(partial), _ptr(sink), _ptr(gate),
            ctypes.c_long(gate_stride), _stream()), "latent_attention")
    return out


def _latent_splits(T, B, H, max_q_len, max_kv_len, window):
    """Over how many blocks a row tile's keys are shared out: only where the step's row tiles
    (64 rows each) leave most of the chip idle and there are keys enough, at least four tiles of
    32 to a share, until there are two blocks a compute unit."""
    tiles = (T * H) // 64 + B
    keys = max_kv_len if window <= 0 else min(max_kv_len, window + max_q_len)
    if tiles >= 256 or keys < 256:
        return 1
    return max(1, min(512 // tiles, keys // 128, 32))


MOE_SCORING = {"softmax": 0, "sigmoid": 1, "sigmoid_groups": 2}


def moe_route(h, router, top, tiled=None, scoring="softmax", correction=None, groups=1, keep=1, experts=None):
    """Per token the `top` experts with the largest scores and their weights: h (T, width),
    router (E, width) of h's dtype (`tiled`: its tile-ordered copy, if the caller keeps one). The
    logits are a product with float32 sums and a float32 result; scores, the choice and the weights
    are float32. Returns chosen int32 (T, top), in the order of falling score (the lowest index
    among equals), and weights float32 (T, top) = score / (sum of the chosen scores + 1e-20) for
    `scoring` "softmax" (scores = softmax over all experts); with "sigmoid" every expert's score is
    sigmoid(z) for itself and the weights are the chosen scores as they are. With "sigmoid_groups" the
    choice goes by sigmoid(z) + correction (`correction` float32 (E,)) and only among the experts of `keep`
    of the `groups` equal groups of neighbouring experts, those groups whose two largest such scores sum
    highest; the weights are sigmoid(z) of the chosen, without the correction.

    `experts`: the router's first `experts` rows are the experts'; what further rows it has are other
    numbers per token that ride on the same product (a gate, say), and their float32 results come back
    as a third value, (T, rows - experts) with rows apart."""
    _dev(h, router, correction)
    _need(scoring in MOE_SCORING, "scoring is softmax or sigmoid")
    _need(h.dim() == 2 and router.dim() == 2 and h.shape[1] == router.shape[1] and h.dtype in _DT
          and router.dtype == h.dtype, "h (T, width) and router (E, width) of one dtype")
    T, rows = h.shape[0], router.shape[0]
    E = rows if experts is None else int(experts)
    _need(1 <= E <= rows and 1 <= top <= E, "experts must lie in 1..rows of the router, top in 1..experts")
    if scoring == "sigmoid_groups":
        _need(correction is not None, "the grouped choice needs a correction")
        _f32(correction, (E,), "correction")
        _need(groups >= 1 and E % groups == 0 and 1 <= keep <= groups and top <= keep * (E // groups),
              "groups divide the experts, keep lies in 1..groups, and the kept groups hold at least top experts")
    else:
        _need(correction is None and groups == 1 and keep == 1, "a correction and groups belong to sigmoid_groups")
    chosen = torch.empty((T, top), dtype=torch.int32, device=h.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=h.device)
    logits = None
    if T:
        logits = linear(h, router, out_dtype=torch.float32, tiled=tiled)
        _check(library("moe").q3_moe_pick(_ptr(logits), ctypes.c_long(rows), T, E, top, MOE_SCORING[scoring],
                                          _ptr(correction), int(groups), int(keep), _ptr(chosen), _ptr(weights),
                                          _stream()), "moe_route")
    if experts is None:
        return chosen, weights
    if logits is None:
        logits = torch.empty((0, rows), dtype=torch.float32, device=h.device)
    return chosen, weights, logits[:, E:]


def moe_experts(h, chosen, weights, up, down, shared=None, activation="erf"):
    """sum_k weights[t, k] * down[e] act(up[e] h[t]), e = chosen[t, k], plus `shared[t]` if given:
    h (T, width), up (E, ff, width), down (E, width, ff), shared (T, width); returns (T, width).
    The (token, choice) pairs are put in the order of their experts on the GPU (no number comes
    back to the host), each expert's product runs over its rows in tiles, and a token's sum is
    formed in float32 in the order of its choices, the shared addend last."""
    _dev(h, chosen, weights, up, down, shared)
    T, width = h.shape
    E, ff = up.shape[0], up.shape[1]
    top = chosen.shape[1]
    _need(h.dtype in _DT and up.dtype == h.dtype and down.dtype == h.dtype and up.shape == (E, ff, width)
          and down.shape == (E, width, ff), "up (E, ff, width) and down (E, width, ff) of h's dtype")
    _need(chosen.shape == (T, top) and chosen.dtype == torch.int32 and weights.shape == (T, top)
          and weights.dtype == torch.float32, "chosen int32 (T, top), weights float32 (T, top)")
    _need(shared is None or (shared.shape == (T, width) and shared.dtype == h.dtype), "shared (T, width)")
    _need(activation in GELU_KINDS, "activation erf or tanh")
    out = torch.empty((T, width), dtype=h.dtype, device=h.device)
    if not T:
        return out
    lib = library("moe")
    P = T * top
    # bfloat16 with inner sizes in steps of 32: the matrix-core kernel over tiles of 64 slots;
    # anything else: float32 multiply-adds over tiles of 16
    cores = h.dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0
    # experts with a hundred rows or more each (prompts): tiles of 128 through shared memory
    # (with inner sizes in steps of 64: tiles of 256 by the dense path's copies and stages)
    many = 3 if width % 64 == 0 and ff % 64 == 0 else 2
    tile_rows = lib.q3_moe_tile_rows((many if P >= 96 * E else 1) if cores else 0)
    tiles, pair_of_slot, slot_of_pair = _moe_book(lib, chosen, E, tile_rows)
    stream = _stream()
    hidden = torch.empty((P, ff), dtype=h.dtype, device=h.device)
    y = torch.empty((P, width), dtype=h.dtype, device=h.device)
    if cores:
        _check(lib.q3_moe_linear_mma(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(up), _ptr(hidden), *tiles, ff, width,
                                     GELU_KINDS[activation], tile_rows, stream), "moe_linear")
        _check(lib.q3_moe_linear_mma(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff,
                                     -1, tile_rows, stream), "moe_linear")
    else:
        _check(lib.q3_moe_linear(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(up), _ptr(hidden), *tiles, ff, width,
                                 GELU_KINDS[activation], _DT[h.dtype], stream), "moe_linear")
        _check(lib.q3_moe_linear(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff, -1,
                                 _DT[h.dtype], stream), "moe_linear")
    _check(lib.q3_moe_combine(_ptr(y), _ptr(slot_of_pair), _ptr(weights), _ptr(shared), None, ctypes.c_long(0), _ptr(out),
                              T, width, top, _DT[h.dtype], stream), "moe_combine")
    return out


def _moe_book(lib, chosen, E, tile_rows):
    """The (token, choice) pairs in the order of their experts: the launch arguments that name the tiles,
    and which pair sits in which slot and the other way round."""
    P = chosen.numel()
    max_tiles = -(-P // tile_rows) + E
    book = torch.empty((E + 1 + 2 * P + 2 * max_tiles + 1,), dtype=torch.int32, device=chosen.device)
    offsets, pair_of_slot, slot_of_pair = book[:E + 1], book[E + 1:E + 1 + P], book[E + 1 + P:E + 1 + 2 * P]
    at = E + 1 + 2 * P
    tile_expert, tile_first, n_tiles = book[at:at + max_tiles], book[at + max_tiles:at + 2 * max_tiles], book[at + 2 * max_tiles:]
    _check(lib.q3_moe_align(_ptr(chosen), P, E, tile_rows, _ptr(offsets), _ptr(pair_of_slot), _ptr(slot_of_pair),
                            _ptr(tile_expert), _ptr(tile_first), _ptr(n_tiles), _stream()), "moe_align")
    return (_ptr(tile_expert), _ptr(tile_first), _ptr(offsets), _ptr(n_tiles), max_tiles), pair_of_slot, slot_of_pair


def moe_gated_experts(h, chosen, weights, gate_up, down, limit, slope):
    """sum_k down[e] y, y = glu(gate_up[e] (weights[t, k] h[t])), e = chosen[t, k]: experts that are gated
    units with clamped branches (`glu_clamped`), whose weight multiplies the expert's input, not its
    result. h (T, width), gate_up (E, 2 ff, width) with rows 2j the gate's and 2j + 1 the other branch's,
    down (E, width, ff); returns (T, width). The weight enters behind the first product, which is
    linear in its input, in float32 and before the clamps; a token's sum is formed in float32 in the
    order of its choices."""
    _dev(h, chosen, weights, gate_up, down)
    T, width = h.shape
    E, ff = down.shape[0], down.shape[2]
    top = chosen.shape[1]
    _need(h.dtype in _DT and gate_up.dtype == h.dtype and down.dtype == h.dtype and gate_up.shape == (E, 2 * ff, width)
          and down.shape == (E, width, ff), "gate_up (E, 2 ff, width) and down (E, width, ff) of h's dtype")
    _need(chosen.shape == (T, top) and chosen.dtype == torch.int32 and weights.shape == (T, top)
          and weights.dtype == torch.float32 and weights.is_contiguous(), "chosen int32 (T, top), weights float32 (T, top)")
    out = torch.empty((T, width), dtype=h.dtype, device=h.device)
    if not T:
        return out
    lib = library("moe")
    P = T * top
    cores = h.dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0
    many = 3 if width % 64 == 0 and ff % 64 == 0 else 2
    tile_rows = lib.q3_moe_tile_rows((many if P >= 96 * E else 1) if cores else 0)
    tiles, pair_of_slot, slot_of_pair = _moe_book(lib, chosen, E, tile_rows)
    both = torch.empty((P, 2 * ff), dtype=h.dtype, device=h.device)
    y = torch.empty((P, width), dtype=h.dtype, device=h.device)
    stream = _stream()
    if cores:
        _check(lib.q3_moe_linear_mma(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(gate_up), _ptr(both), *tiles, 2 * ff, width,
                                     -1, tile_rows, stream), "moe_linear")
    else:
        _check(lib.q3_moe_linear(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(gate_up), _ptr(both), *tiles, 2 * ff, width, -1,
                                 _DT[h.dtype], stream), "moe_linear")
    hidden = glu_clamped(both, limit, slope, scale=weights.view(-1), scale_index=pair_of_slot)
    if cores:
        _check(lib.q3_moe_linear_mma(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff,
                                     -1, tile_rows, stream), "moe_linear")
    else:
        _check(lib.q3_moe_linear(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff, -1,
                                 _DT[h.dtype], stream), "moe_linear")
    _check(lib.q3_moe_combine(_ptr(y), _ptr(slot_of_pair), None, None, None, ctypes.c_long(0), _ptr(out), T, width, top,
                              _DT[h.dtype], stream), "moe_combine")
    return out


_MOE_ACT_GATED = 2      # the experts' product kernels: epilogue codes from here on are gated units, in the order of GATE_KINDS


def moe_glu_experts(h, chosen, weights, gate_up, down, activation="silu", shared=None, shared_gate=None):
    """sum_k weights[t, k] * down[e] (act(gate[e] h[t]) * (up[e] h[t])), e = chosen[t, k]: experts that are
    gated units without biases, weighted on their results. h (T, width), gate_up (E, 2 ff, width) with rows
    2j the gate's and 2j + 1 the other branch's, down (E, width, ff), `activation` one of `GATE_KINDS`;
    `shared` (T, width) is added last, multiplied by sigmoid(shared_gate[t]) when `shared_gate` (float32
    (T,) or (T, 1), rows possibly apart: a logit per token) is given. Returns (T, width). The pairs are
    sorted by expert on the GPU as in `moe_experts`; the gated unit is the epilogue of the first product,
    from its float32 sums; a token's sum is formed in float32 in the order of its choices."""
    _dev(h, chosen, weights, gate_up, down, shared)
    T, width = h.shape
    E, ff = down.shape[0], down.shape[2]
    top = chosen.shape[1]
    _need(h.dtype in _DT and gate_up.dtype == h.dtype and down.dtype == h.dtype and gate_up.shape == (E, 2 * ff, width)
          and down.shape == (E, width, ff), "gate_up (E, 2 ff, width) and down (E, width, ff) of h's dtype")
    _need(chosen.shape == (T, top) and chosen.dtype == torch.int32 and weights.shape == (T, top)
          and weights.dtype == torch.float32 and weights.is_contiguous(), "chosen int32 (T, top), weights float32 (T, top)")
    _need(shared is None or (shared.shape == (T, width) and shared.dtype == h.dtype), "shared (T, width)")
    _need(activation in GATE_KINDS, "activation is one of %s" % ", ".join(sorted(GATE_KINDS)))
    gate_stride = 0
    if shared_gate is not None:
        _need(shared is not None and shared_gate.is_cuda and shared_gate.dtype == torch.float32
              and shared_gate.numel() == T and shared_gate.shape[0] == T, "shared_gate float32, one logit per token")
        gate_stride = shared_gate.stride(0)
    out = torch.empty((T, width), dtype=h.dtype, device=h.device)
    if not T:
        return out
    lib = library("moe")
    P = T * top
    cores = h.dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0
    many = 3 if width % 64 == 0 and ff % 64 == 0 else 2
    tile_rows = lib.q3_moe_tile_rows((many if P >= 96 * E else 1) if cores else 0)
    tiles, pair_of_slot, slot_of_pair = _moe_book(lib, chosen, E, tile_rows)
    hidden = torch.empty((P, ff), dtype=h.dtype, device=h.device)
    y = torch.empty((P, width), dtype=h.dtype, device=h.device)
    stream = _stream()
    gated = _MOE_ACT_GATED + GATE_KINDS[activation]      # the gated unit is the first product's epilogue, on unrounded sums
    if cores:
        _check(lib.q3_moe_linear_mma(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(gate_up), _ptr(hidden), *tiles, 2 * ff, width,
                                     gated, tile_rows, stream), "moe_linear")
    else:
        _check(lib.q3_moe_linear(_ptr(h), _ptr(pair_of_slot), 1, top, _ptr(gate_up), _ptr(hidden), *tiles, 2 * ff, width,
                                 gated, _DT[h.dtype], stream), "moe_linear")
    if cores:
        _check(lib.q3_moe_linear_mma(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff,
                                     -1, tile_rows, stream), "moe_linear")
    else:
        _check(lib.q3_moe_linear(_ptr(hidden), _ptr(pair_of_slot), 0, 1, _ptr(down), _ptr(y), *tiles, width, ff, -1,
                                 _DT[h.dtype], stream), "moe_linear")
    _check(lib.q3_moe_combine(_ptr(y), _ptr(slot_of_pair), _ptr(weights), _ptr(shared), _ptr(shared_gate),
                              ctypes.c_long(gate_stride), _ptr(out), T, width, top, _DT[h.dtype], stream), "moe_combine")
    return out


# ---- a residual in several streams; the recurrent mixers; attention with capped scores ----

def _f32(t, shape, what):
    _need(t.dtype == torch.float32 and tuple(t.shape) == tuple(shape) and t.is_contiguous() and t.is_cuda,
          "%s must be float32 %s on the GPU, contiguous" % (what, tuple(shape)))


def _rows_view(t, what):
    """A 2-D tensor whose rows may lie apart (a stretch of columns of a wider tensor)."""
    _need(t.is_cuda and t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1) and t.dtype in _DT,
          "%s must be (rows, n) on the GPU with its columns side by side" % what)
    return t.stride(0)


def _sequences(slots, cu_seqlens_q, state, numbers, what):
    _need(slots.dtype == torch.int32 and cu_seqlens_q.dtype == torch.int32 and slots.dim() == 1
          and cu_seqlens_q.shape == (slots.shape[0] + 1,), "slots int32 (B,), cu_seqlens_q int32 (B + 1,)")
    _dev(slots, cu_seqlens_q)
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == numbers
          and (numbers == 1 or state.stride(1) == 1),
          "%s: the state must be float32 (slots, %d) on the GPU with its columns side by side" % (what, numbers))
    return slots.shape[0]


def embed_streams(ids, table, copies):
    """out[t, s, :] = float32(table[ids[t], :]) for s < copies: a residual that starts as equal streams."""
    _dev(ids, table)
    _need(ids.dtype == torch.int32 and ids.dim() == 1, "ids must be int32 (T,)")
    _need(table.dim() == 2 and table.dtype in _DT and 1 <= copies <= 8, "table (V, W) bfloat16 or float32; 1 to 8 copies")
    T, (V, W) = ids.shape[0], table.shape
    out = torch.empty((T, copies, W), dtype=torch.float32, device=table.device)
    if T:
        _check(library("hyper").q3_embed_streams(_ptr(ids), _ptr(table), _ptr(out), T, copies, W, V, _DT[table.dtype],
                                                 _stream()), "embed_streams")
    return out


def hyper_norm(x, weight, eps, out_dtype, read=None, delta=None, mix=None, write=None, rows=None, write_back=True):
    """Layer norm of a float32 residual held in streams, x (T, S, W), behind an addend that enters
    all streams at once. For each output row r (source row s = rows[r], or r):

    with `delta` (T, W, activation dtype), `mix` (S, S) indexed [from, to] and `write` (S,):
    x[s, t] <- sum_f mix[f, t] x[s, f] + write[t] * delta[s] for all t from the old streams, stored if
    `write_back` and `rows` is None; u = sum_f read[f] x[s, f] (`read` None: the plain sum);
    out[r] = (u - mean(u)) * rsqrt(mean((u - mean(u))^2) + eps) * weight, rounded once to `out_dtype`.
    With `weight` None only the streams are brought up to date and None is returned."""
    _dev(x, weight, delta, mix, write, read, rows)
    _need(x.dim() == 3 and x.dtype == torch.float32 and 1 <= x.shape[1] <= 8, "x must be float32 (T, S, W), S at most 8")
    T, S, W = x.shape
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    if weight is not None:
        _f32(weight, (W,), "weight")
    if read is not None:
        _f32(read, (S,), "read")
    if delta is not None:
        _need(delta.shape == (T, W) and delta.dtype == out_dtype, "delta must be (T, W) of the activation dtype")
        _need(mix is not None and write is not None, "a delta comes with mix and write")
        _f32(mix, (S, S), "mix")
        _f32(write, (S,), "write")
    n_out = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1, "rows must be int32 (R,)")
        n_out = rows.shape[0]
    _need(weight is not None or rows is None, "without a weight there is no output")
    out = torch.empty((n_out, W), dtype=out_dtype, device=x.device) if weight is not None else None
    if n_out:
        _check(library("hyper").q3_hyper_norm(
            _ptr(x), _ptr(delta), _ptr(mix), _ptr(write), _ptr(read), _ptr(weight), _ptr(rows), _ptr(out), n_out, S, W,
            ctypes.c_float(eps), _DT[out_dtype], 1 if (write_back and rows is None and delta is not None) else 0,
            _stream()), "hyper_norm")
    return out


def causal_conv(x, weight, bias, state, slots, cu_seqlens_q, seq_index, activation=None, out_dtype=None, in_bias=None,
                max_q_len=0):
    """A causal convolution per channel over a packed step, continued from each sequence's state.

    x (T, C), rows possibly apart; weight float32 (C, taps), the last tap the current token's; bias
    float32 (C,); `in_bias` float32 (C,) is added to x first. state float32 (slots, (taps - 1) * C):
    a sequence's last taps - 1 inputs, oldest first (zeros for a fresh sequence), brought up to
    date. `activation`: None or "silu". Returns (T, C) of `out_dtype` (x's by default). `max_q_len` 1
    says that every sequence brings one row: output and new tail are then one kernel."""
    stride = _rows_view(x, "x")
    T, C = x.shape
    taps = weight.shape[1] if weight.dim() == 2 else 0
    _f32(weight, (C, taps), "weight")
    _f32(bias, (C,), "bias")
    if in_bias is not None:
        _f32(in_bias, (C,), "in_bias")
    _need(1 <= taps <= 8 and activation in (None, "silu"), "1 to 8 taps; activation None or silu")
    B = _sequences(slots, cu_seqlens_q, state, (taps - 1) * C, "causal_conv")
    _need(seq_index.dtype == torch.int32 and seq_index.shape == (T,), "seq_index must be int32 (T,)")
    _dev(seq_index)
    out_dtype = out_dtype or x.dtype
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    out = torch.empty((T, C), dtype=out_dtype, device=x.device)
    if T:
        _check(library("recurrent").q3_causal_conv(
            _ptr(x), ctypes.c_long(stride), _ptr(in_bias), _ptr(weight), _ptr(bias), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(seq_index), _ptr(out), T, B, C, taps,
            1 if activation == "silu" else 0, 1 if (max_q_len == 1 and T == B) else 0, _DT[x.dtype], _DT[out_dtype],
            _stream()), "causal_conv")
    return out


CHUNKED_FROM = 9      # a step whose longest sequence brings this many rows takes the recurrences' chunked kernels


def mamba2_scan(xbc, dt, dt_bias, a_log, d_skip, state, slots, cu_seqlens_q, heads, vdim, n_state, groups, max_q_len=1):
    """The Mamba-2 recurrence over a packed step. xbc (T, heads vdim + 2 groups n_state), contiguous,
    rows [x | B | C]; dt (T, heads), rows possibly apart, same dtype; dt_bias, a_log, d_skip float32
    (heads,). Per head h of group g = h // (heads / groups), with step = softplus(dt + dt_bias):
    S <- exp(-exp(a_log) step) S + step B x^T, y = S^T C + d_skip x. state float32 (slots,
    heads n_state vdim) laid out (head, n, column), continued and brought up to date. Returns y
    float32 (T, heads vdim). `max_q_len`: the rows of the step's longest sequence; from `CHUNKED_FROM` on
    the sequences are worked through in chunks of 64 rows, all chunks at once, instead of row by row."""
    _dev(xbc, dt_bias, a_log, d_skip)
    T = xbc.shape[0]
    _need(xbc.dim() == 2 and xbc.dtype in _DT and xbc.shape[1] == heads * vdim + 2 * groups * n_state,
          "xbc must be (T, heads vdim + 2 groups n_state)")
    stride = _rows_view(dt, "dt")
    _need(dt.shape == (T, heads) and dt.dtype == xbc.dtype, "dt must be (T, heads) of xbc's dtype")
    for t, what in ((dt_bias, "dt_bias"), (a_log, "a_log"), (d_skip, "d_skip")):
        _f32(t, (heads,), what)
    _need(heads % groups == 0 and n_state <= 256, "groups must divide heads; n_state at most 256")
    B = _sequences(slots, cu_seqlens_q, state, heads * n_state * vdim, "mamba2_scan")
    y = torch.empty((T, heads * vdim), dtype=torch.float32, device=xbc.device)
    if T and max_q_len >= CHUNKED_FROM:
        lib = library("recurrent")
        lib.q3_chunked_workspace.restype = ctypes.c_long
        work = torch.empty(lib.q3_chunked_workspace(T, B, heads, groups, n_state, vdim), dtype=torch.float32, device=xbc.device)
        _check(lib.q3_mamba2_chunked(
            _ptr(xbc), _ptr(dt), ctypes.c_long(stride), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(y), _ptr(work), T, B, int(max_q_len),
            heads, vdim, n_state, groups, _DT[xbc.dtype], _stream()), "mamba2_scan")
        return y
    if T:
        _check(library("recurrent").q3_mamba2_scan(
            _ptr(xbc), _ptr(dt), ctypes.c_long(stride), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(y), B, heads, vdim, n_state, groups,
            _DT[xbc.dtype], _stream()), "mamba2_scan")
    return y


def gated_rmsnorm(y, gate, weight, groups, eps, out_dtype):
    """v = y * silu(gate); out = v * rsqrt(mean(v^2) + eps) * weight, the mean taken over each of
    `groups` equal parts of a row. y float32 (T, n) contiguous, gate (T, n) of `out_dtype`, rows
    possibly apart, weight float32 (n,)."""
    _dev(y, weight)
    _need(y.dim() == 2 and y.dtype == torch.float32, "y must be float32 (T, n)")
    T, n = y.shape
    stride = _rows_view(gate, "gate")
    _need(gate.shape == (T, n) and gate.dtype == out_dtype and out_dtype in _DT, "gate must be (T, n) of out_dtype")
    _f32(weight, (n,), "weight")
    _need(groups >= 1 and n % groups == 0, "groups must divide the row")
    out = torch.empty((T, n), dtype=out_dtype, device=y.device)
    if T:
        _check(library("hyper").q3_gated_rmsnorm(_ptr(y), _ptr(gate), ctypes.c_long(stride), _ptr(weight), _ptr(out), T, n,
                                                 groups, ctypes.c_float(eps), _DT[out_dtype], _stream()), "gated_rmsnorm")
    return out


def block_gates(u, weights, biases):
    """out[g, t, b bw + o] = sigmoid(biases[g, b, o] + sum_i weights[g, b, i, o] u[t, b bw + i]): two gates
    from block-diagonal matrices, float32 throughout. u (T, width), weights (2, blocks, bw, bw) indexed
    (gate, block, in, out), biases (2, blocks, bw). Returns (2, T, width)."""
    _dev(u, weights, biases)
    _need(u.dim() == 2 and u.dtype == torch.float32, "u must be float32 (T, width)")
    T, width = u.shape
    _need(weights.dim() == 4 and weights.shape[0] == 2 and weights.shape[2] == weights.shape[3]
          and weights.shape[1] * weights.shape[2] == width, "weights must be (2, blocks, bw, bw) with blocks bw = width")
    blocks, bw = weights.shape[1], weights.shape[2]
    _f32(weights, (2, blocks, bw, bw), "weights")
    _f32(biases, (2, blocks, bw), "biases")
    out = torch.empty((2, T, width), dtype=torch.float32, device=u.device)
    if T:
        _check(library("recurrent").q3_block_gates(_ptr(u), _ptr(weights), _ptr(biases), _ptr(out), T, width, blocks,
                                                   _stream()), "block_gates")
    return out


def rglru_scan(u, gates, rate, y, y_bias, state, slots, cu_seqlens_q, out_dtype, max_q_len=1):
    """The real-gated linear recurrence over a packed step, float32: with r = gates[0], i = gates[1],
    a = exp(-rate r): S <- a S + sqrt(1 - a^2) i u; out = S * gelu_tanh(y + y_bias), rounded once to
    `out_dtype`. u (T, width) and gates (2, T, width) float32 contiguous, y float32 (T, width) with
    rows possibly apart, rate and y_bias float32 (width,), state float32 (slots, width). A step whose
    longest sequence (`max_q_len`) passes 64 rows is worked through in segments of 64 rows at once."""
    _dev(u, gates, rate, y_bias)
    _need(u.dim() == 2 and u.dtype == torch.float32, "u must be float32 (T, width)")
    T, width = u.shape
    _f32(gates, (2, T, width), "gates")
    _f32(rate, (width,), "rate")
    _f32(y_bias, (width,), "y_bias")
    stride = _rows_view(y, "y")
    _need(y.shape == (T, width) and y.dtype == torch.float32 and out_dtype in _DT, "y must be float32 (T, width)")
    B = _sequences(slots, cu_seqlens_q, state, width, "rglru_scan")
    out = torch.empty((T, width), dtype=out_dtype, device=u.device)
    if T and max_q_len > 64:
        work = torch.empty((2 * (T // 64 + B) * width,), dtype=torch.float32, device=u.device)
        _check(library("recurrent").q3_rglru_chunked(
            _ptr(u), _ptr(gates), _ptr(rate), _ptr(y), ctypes.c_long(stride), _ptr(y_bias), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(out), _ptr(work), T, B, int(max_q_len),
            width, _DT[out_dtype], _stream()), "rglru_scan")
        return out
    if T:
        _check(library("recurrent").q3_rglru_scan(
            _ptr(u), _ptr(gates), _ptr(rate), _ptr(y), ctypes.c_long(stride), _ptr(y_bias), _ptr(state),
            ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(out), T, B, width, _DT[out_dtype],
            _stream()), "rglru_scan")
    return out


def retention_scan(qkvg, heads, dim, vdim, inv_freq, positions, decay, k_scale, eps, state, slots, cu_seqlens_q, out_dtype,
                   max_q_len=1, log_decay=None):
    """Retention over a packed step. qkvg (T, 2 heads dim + 2 heads vdim) contiguous, rows
    [q | k | v | g]. q and k turn by the position over their first 2 len(inv_freq) numbers, pairs
    (i, i + len(inv_freq)), angle = position * inv_freq[i] in float32 (`inv_freq` None: no rotation);
    k is multiplied by `k_scale`. Per head S <- decay S + k v^T, o = S^T q; o is divided by the root
    mean square of the head's vdim numbers (eps inside the root) and multiplied by silu(g). state
    float32 (slots, heads dim vdim) laid out (head, dim, column). Returns (T, heads vdim).
    `max_q_len` as for `mamba2_scan`; the chunked kernels take the decays' logarithms, `log_decay`
    float32 (heads,), formed here if not given."""
    _dev(qkvg, inv_freq, positions, decay)
    T = qkvg.shape[0]
    _need(qkvg.dim() == 2 and qkvg.dtype in _DT and qkvg.dtype == out_dtype
          and qkvg.shape[1] == 2 * heads * dim + 2 * heads * vdim, "qkvg must be (T, 2 heads dim + 2 heads vdim) of out_dtype")
    half = 0
    if inv_freq is not None:
        half = inv_freq.shape[0]
        _f32(inv_freq, (half,), "inv_freq")
    _need(2 * half <= dim and dim <= 256, "the rotation fits the head; dim at most 256")
    _need(positions.dtype == torch.int32 and positions.shape == (T,), "positions must be int32 (T,)")
    _f32(decay, (heads,), "decay")
    B = _sequences(slots, cu_seqlens_q, state, heads * dim * vdim, "retention_scan")
    out = torch.empty((T, heads * vdim), dtype=out_dtype, device=qkvg.device)
    if T and max_q_len >= CHUNKED_FROM:
        lib = library("recurrent")
        lib.q3_chunked_workspace.restype = ctypes.c_long
        if log_decay is None:
            log_decay = torch.log(decay.double()).float()
        _f32(log_decay, (heads,), "log_decay")
        work = torch.empty(lib.q3_chunked_workspace(T, B, heads, heads, dim, vdim), dtype=torch.float32, device=qkvg.device)
        raw = torch.empty((T, heads * vdim), dtype=torch.float32, device=qkvg.device)
        _check(lib.q3_retention_chunked(
            _ptr(qkvg), _ptr(inv_freq), half, _ptr(positions), _ptr(log_decay), ctypes.c_float(k_scale),
            ctypes.c_float(eps), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(out),
            _ptr(work), _ptr(raw), T, B, int(max_q_len), heads, dim, vdim, _DT[out_dtype], _stream()), "retention_scan")
        return out
    if T:
        raw = torch.empty((T, heads * vdim), dtype=torch.float32, device=qkvg.device)
        _check(library("recurrent").q3_retention_scan(
            _ptr(qkvg), _ptr(inv_freq), half, _ptr(positions), _ptr(decay), ctypes.c_float(k_scale), ctypes.c_float(eps),
            _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(out), _ptr(raw), T, B,
            heads, dim, vdim, _DT[out_dtype], _stream()), "retention_scan")
    return out


def softcap_prepare(rows, bias, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, inv_freq, positions, seq_index,
                    out_dtype, block_table=None, k_cache=None, v_cache=None, values_transposed=False):
    """Queries, keys and values of a step from the float32 rows of their joint product.

    rows float32 (T, n), n >= heads dim + kv_heads dim + kv_heads vdim, laid out [q | k | v | ...];
    bias float32 over q, k and v is added (None: projections without biases); q and k are each divided by the root mean square of the
    whole projection and multiplied by `q_weight` (heads dim) and `k_weight` (kv_heads dim); the
    first 2 len(inv_freq) numbers of every head turn in pairs (2i, 2i + 1) by position * inv_freq[i].
    Returns q (T, heads, dim) of `out_dtype`; with a cache, keys (pages, kv_heads, page, dim) and
    values (pages, kv_heads, page, vdim), or (pages, kv_heads, vdim, page) with `values_transposed`,
    receive the tokens at their positions."""
    _dev(bias, q_weight, k_weight, inv_freq, positions, seq_index, block_table, k_cache, v_cache)
    _need(rows.is_cuda and rows.dim() == 2 and rows.dtype == torch.float32 and rows.stride(1) == 1, "rows must be float32 (T, n)")
    T = rows.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    _need(rows.shape[1] >= nq + nk + nv and heads % kv_heads == 0, "rows hold q, k and v; kv_heads divides heads")
    if bias is not None:
        _f32(bias, (nq + nk + nv,), "bias")
    _f32(q_weight, (nq,), "q_weight")
    _f32(k_weight, (nk,), "k_weight")
    half = 0
    if inv_freq is not None:
        half = inv_freq.shape[0]
        _f32(inv_freq, (half,), "inv_freq")
    _need(2 * half <= dim and out_dtype in _DT, "the rotation fits the head")
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and seq_index.dtype == torch.int32
          and seq_index.shape == (T,), "positions and seq_index must be int32 (T,)")
    page = width = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None and block_table.dtype == torch.int32 and block_table.dim() == 2,
              "a key cache comes with a value cache and an int32 block table")
        page, width = k_cache.shape[2], block_table.shape[1]
        _need(k_cache.dim() == 4 and k_cache.shape[1:] == (kv_heads, page, dim) and v_cache.dim() == 4
              and v_cache.shape[1:] == ((kv_heads, vdim, page) if values_transposed else (kv_heads, page, vdim))
              and k_cache.dtype == out_dtype and v_cache.dtype == out_dtype,
              "keys (pages, kv_heads, page, dim) and values (pages, kv_heads, page, vdim) of out_dtype")
    q = torch.empty((T, heads, dim), dtype=out_dtype, device=rows.device)
    if T:
        _check(library("softcap").q3_softcap_prepare(
            _ptr(rows), ctypes.c_long(rows.stride(0)), _ptr(bias), _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps),
            _ptr(inv_freq), half, _ptr(positions), _ptr(seq_index), _ptr(block_table), width, _ptr(k_cache), _ptr(v_cache),
            page, _ptr(q), T, heads, kv_heads, dim, vdim, 1 if values_transposed else 0, _DT[out_dtype], _stream()),
            "softcap_prepare")
    return q


def headnorm_prepare(rows, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, positions, seq_index, out_dtype,
                     block_table=None, k_cache=None, v_cache=None, values_transposed=False):
    """Queries, keys and values of a step from the float32 rows of their joint product, with a norm per
    head and no rotation.

    rows float32 (T, n) laid out [q: heads dim | k: kv_heads dim | v: kv_heads vdim | ...]; every head
    of q and of k is divided by its own root mean square (eps inside the root) and multiplied by
    `q_weight` or `k_weight`, float32 (dim,), shared by the heads. Returns q (T, heads, dim) of
    `out_dtype`; keys and values go to their positions in the cache, laid out as for
    `softcap_prepare`. With `kv_heads` 0 the rows hold no keys and values (a layer that reads
    another layer's) and nothing is written."""
    _dev(q_weight, k_weight, positions, seq_index, block_table, k_cache, v_cache)
    _need(rows.is_cuda and rows.dim() == 2 and rows.dtype == torch.float32 and rows.stride(1) == 1, "rows must be float32 (T, n)")
    T = rows.shape[0]
    _need(heads > 0 and kv_heads >= 0 and (kv_heads == 0 or heads % kv_heads == 0), "kv_heads divides heads (or is 0)")
    _need(rows.shape[1] >= heads * dim + kv_heads * (dim + vdim), "rows hold q, k and v")
    _f32(q_weight, (dim,), "q_weight")
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and seq_index.dtype == torch.int32
          and seq_index.shape == (T,), "positions and seq_index must be int32 (T,)")
    page = width = 0
    if kv_heads:
        _f32(k_weight, (dim,), "k_weight")
        _need(k_cache is not None and v_cache is not None and block_table is not None and block_table.dtype == torch.int32
              and block_table.dim() == 2, "keys of its own need a key cache, a value cache and an int32 block table")
        page, width = k_cache.shape[2], block_table.shape[1]
        _need(k_cache.dim() == 4 and k_cache.shape[1:] == (kv_heads, page, dim) and v_cache.dim() == 4
              and v_cache.shape[1:] == ((kv_heads, vdim, page) if values_transposed else (kv_heads, page, vdim))
              and k_cache.dtype == out_dtype and v_cache.dtype == out_dtype and k_cache.is_contiguous()
              and v_cache.is_contiguous(),
              "keys (pages, kv_heads, page, dim) and values (pages, kv_heads, page, vdim) of out_dtype")
    q = torch.empty((T, heads, dim), dtype=out_dtype, device=rows.device)
    if T:
        _check(library("softcap").q3_headnorm_prepare(
            _ptr(rows), ctypes.c_long(rows.stride(0)), _ptr(q_weight), _ptr(k_weight) if kv_heads else None,
            ctypes.c_float(eps), _ptr(positions), _ptr(seq_index), _ptr(block_table) if kv_heads else None, width,
            _ptr(k_cache) if kv_heads else None, _ptr(v_cache) if kv_heads else None, page, _ptr(q), T, heads, kv_heads,
            dim, vdim, 1 if values_transposed else 0, _DT[out_dtype], _stream()), "headnorm_prepare")
    return q


def channel_delta(conv, b_logits, a_logits, gate, dt_bias, a_log, norm_weight, eps, unit_eps, state, slots, cu_seqlens_q,
                  heads, kv_heads, dim, vdim, out_dtype):
    """The gated delta rule with a decay per head and key channel over a packed step, float32.

    conv float32 (T, 2 kv_heads dim + heads vdim) contiguous: [q | k | v] behind their convolutions and
    activations; head h reads q and k of group h // (heads / kv_heads). b_logits (T, heads), a_logits
    (T, heads dim) and gate (T, heads vdim): float32, rows possibly apart. q and k become unit vectors
    per head, x / sqrt(sum(x^2) + unit_eps), q also times dim^(-1/2); beta = sigmoid(b_logits);
    g = exp(-exp(a_log[h]) softplus(a_logits + dt_bias)), a number per head and key channel. Per head

        S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;

    o is divided by the root mean square of the head's vdim numbers (eps inside the root), multiplied
    by `norm_weight` (vdim,) and by sigmoid(gate). state float32 (slots, heads vdim dim) laid out (head,
    column, row), continued and brought up to date. Returns (T, heads vdim) of `out_dtype`."""
    _dev(conv, dt_bias, a_log, norm_weight)
    T = conv.shape[0]
    _need(heads > 0 and kv_heads > 0 and heads % kv_heads == 0 and 0 < dim <= 256 and vdim > 0,
          "kv_heads divides heads; dim at most 256")
    _f32(conv, (T, 2 * kv_heads * dim + heads * vdim), "conv")
    for t, n, what in ((b_logits, heads, "b_logits"), (a_logits, heads * dim, "a_logits"), (gate, heads * vdim, "gate")):
        _rows_view(t, what)
        _need(t.shape == (T, n) and t.dtype == torch.float32, "%s must be float32 (T, %d)" % (what, n))
    _f32(dt_bias, (heads * dim,), "dt_bias")
    _f32(a_log, (heads,), "a_log")
    _f32(norm_weight, (vdim,), "norm_weight")
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    B = _sequences(slots, cu_seqlens_q, state, heads * dim * vdim, "channel_delta")
    out = torch.empty((T, heads * vdim), dtype=out_dtype, device=conv.device)
    if T:
        lib = library("delta")
        lib.q3_channel_delta_workspace.restype = ctypes.c_long
        work = torch.empty(lib.q3_channel_delta_workspace(T, heads, dim, vdim), dtype=torch.float32, device=conv.device)
        _check(lib.q3_channel_delta(
            _ptr(conv), _ptr(b_logits), ctypes.c_long(b_logits.stride(0)), _ptr(a_logits), ctypes.c_long(a_logits.stride(0)),
            _ptr(gate), ctypes.c_long(gate.stride(0)), _ptr(dt_bias), _ptr(a_log), _ptr(norm_weight), ctypes.c_float(eps),
            ctypes.c_float(unit_eps), _ptr(state), ctypes.c_long(state.stride(0)), _ptr(slots), _ptr(cu_seqlens_q), _ptr(out),
            _ptr(work), T, B, heads, kv_heads, dim, vdim, _DT[out_dtype], _stream()), "channel_delta")
    return out


def softcap_attention(q, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, seq_index, positions, max_q_len,
                      max_kv_len, scale, softcap, window=0, gate=None, values_transposed=False, min_q_len=1,
                      max_kv_len_of_many=None, sink=None):
    """Causal softmax attention over a paged cache whose keys and values differ in size.

    q (T, heads, dim); keys (pages, kv_heads, page, dim), values (pages, kv_heads, page, vdim); the
    token at row t of sequence seq_index[t] sits at positions[t] and sees the keys at positions
    j <= positions[t] (with `window` > 0 only the last `window` of them). score = (q . k) scale, then
    softcap * tanh(score / softcap) if softcap > 0; softmax in float32. `gate` float32 (T, heads),
    rows possibly apart: head h's result is multiplied by sigmoid(gate[t, h]). `sink` float32 (heads,):
    head h's softmax has exp(sink[h]) as one more term of its denominator, a key that is always seen, is
    not scaled and has no value. Returns (T, heads vdim).

    With `values_transposed` the values are (pages, kv_heads, vdim, page), and bfloat16 with equal key
    and value sizes of 64 or 128 then runs on the matrix cores, through the kernels of
    `paged_attention` (`min_q_len` and `max_kv_len_of_many` are theirs); everything else takes a
    general kernel of one wavefront per (token, head)."""
    _dev(q, k_cache, v_cache, block_table, seq_index, positions, sink)
    _need(q.dim() == 3 and q.dtype in _DT, "q must be (T, heads, dim)")
    T, H, dim = q.shape
    if sink is not None:
        _f32(sink, (H,), "sink")
    _need(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[3] == dim and k_cache.shape[:2] == v_cache.shape[:2]
          and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "keys (pages, G, page, dim), values (pages, G, page, vdim)")
    G, page = k_cache.shape[1], k_cache.shape[2]
    vdim = v_cache.shape[2] if values_transposed else v_cache.shape[3]
    _need(v_cache.shape[2:] == ((vdim, page) if values_transposed else (page, vdim)), "keys and values differ in their pages")
    _need(H % G == 0 and dim <= 512 and vdim <= 512, "kv heads divide heads; dim and vdim at most 512")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (B, W)")
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and seq_index.dtype == torch.int32
          and seq_index.shape == (T,), "positions and seq_index must be int32 (T,)")
    _need(max_kv_len <= block_table.shape[1] * page, "the block table does not cover the longest sequence")
    stride = 0
    if gate is not None:
        stride = _rows_view(gate, "gate")
        _need(gate.shape == (T, H) and gate.dtype == torch.float32, "gate must be float32 (T, heads)")
    if T and values_transposed and dim == vdim and q.dtype == torch.bfloat16 \
            and library("attention").q3_paged_attention_fast_path(H, G, dim, page, _DT[q.dtype]):
        out = paged_attention(q, H, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, max_q_len, max_kv_len, scale,
                              window=window, min_q_len=min_q_len, max_kv_len_of_many=max_kv_len_of_many, softcap=softcap,
                              sink=sink)
        if gate is not None:
            _check(library("softcap").q3_gate_heads(_ptr(out), _ptr(gate), ctypes.c_long(stride), T, H, vdim,
                                                    _DT[q.dtype], _stream()), "gate_heads")
        return out
    out = torch.empty((T, H * vdim), dtype=q.dtype, device=q.device)
    if T:
        _check(library("softcap").q3_softcap_attention(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(seq_index),
            _ptr(positions), ctypes.c_float(scale), ctypes.c_float(softcap), int(window), _ptr(gate),
            ctypes.c_long(stride), _ptr(out), T, H, G, dim, vdim, page, 1 if values_transposed else 0, _ptr(sink),
            _DT[q.dtype], _stream()), "softcap_attention")
    return out


def scaled_sum(a, alpha, b, beta):
    """alpha * a + beta * b, elementwise in float32, rounded once to the operands' dtype."""
    _dev(a, b)
    _need(a.shape == b.shape and a.dtype == b.dtype and a.dtype in _DT, "a and b must be alike, bfloat16 or float32")
    out = torch.empty_like(a)
    if a.numel():
        _check(library("hyper").q3_scaled_sum(_ptr(a), ctypes.c_float(alpha), _ptr(b), ctypes.c_float(beta), _ptr(out),
                                              ctypes.c_long(a.numel()), _DT[a.dtype], _stream()), "scaled_sum")
    return out


def rope_table(inv_freq, max_positions):
    """table[p] = [cos(p * inv_freq) | sin(p * inv_freq)], float32 (P, 2 * len(inv_freq))."""
    _dev(inv_freq)
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1, "inv_freq must be float32 (D/2,)")
    half = inv_freq.shape[0]
    table = torch.empty((max_positions, 2 * half), dtype=torch.float32, device=inv_freq.device)
    _check(library("rotary").q3_rope_table(
        _ptr(inv_freq), _ptr(table), max_positions, half, _stream()), "rope_table")
    return table


def qk_norm_rope_store(qkv, num_q_heads, num_kv_heads, head_dim, positions, seq_index,
                       q_weight=None, k_weight=None, eps=0.0, table=None,
                       block_table=None, k_cache=None, v_cache=None,
                       cu_seqlens_q=None, kv_lens=None, max_q_len=0, max_kv_len=0):
    """Per-head RMSNorm of q and k, rotation by position, and the cache write, in one pass.

    qkv (T, (Hq + 2 Hkv) D) holds [q heads | k heads | v heads]. q heads are
    normalised with `q_weight`, rotated, and written back in place. k heads
    are normalised with `k_weight`, rotated, and stored; v heads are stored as
    they are. The store goes to page block_table[seq_index[t], pos // page] at
    slot pos % page of a key cache shaped (pages, Hkv, page, D) and a value
    cache shaped (pages, Hkv, D, page); entries below zero are skipped, and
    nothing is stored when no cache is given. Norm and
    rotation are each skipped when their operand is None. The rotation pairs
    element i with i + R/2 over the first R = table.shape[1] elements.
    `cu_seqlens_q`, `kv_lens` (after this step's write) and `max_q_len`
    describe the step's sequences; with them, bfloat16 steps use kernels with
    16-byte accesses that write values page by page. positions must then be
    kv_lens[b] - q_len[b] + i for row i of sequence b, as the step function
    makes them. `max_kv_len`: the step's last position + 1, if the caller knows it;
    a step that passes the end of the rotation table is refused (a position
    the table does not hold would go without its rotation).
    """
    _dev(qkv, positions, seq_index, q_weight, k_weight, table, block_table, k_cache, v_cache,
         cu_seqlens_q, kv_lens)
    if (cu_seqlens_q is None) != (kv_lens is None):
        raise OperandError("cu_seqlens_q and kv_lens are given together or not at all")
    if kv_lens is not None:
        _need(kv_lens.dtype == torch.int32 and cu_seqlens_q.dtype == torch.int32
              and cu_seqlens_q.shape == (kv_lens.shape[0] + 1,) and max_q_len > 0,
              "cu_seqlens_q int32 (B+1,), kv_lens int32 (B,), max_q_len > 0")
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == (Hq + 2 * Hkv) * D and qkv.dtype in _DT,
          "qkv must be (T, (Hq + 2 Hkv) D) bfloat16 or float32")
    T = qkv.shape[0]
    _need(1 <= D <= 512, "head_dim must be in 1..512")
    for t in (positions, seq_index):
        _need(t.dtype == torch.int32 and t.shape == (T,), "positions and seq_index must be int32 (T,)")
    w_dtype = 0
    if (q_weight is None) != (k_weight is None):
        raise OperandError("q_weight and k_weight are given together or not at all")
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype in _DT
              and k_weight.dtype == q_weight.dtype, "norm weights must be (D,), same dtype")
        w_dtype = _DT[q_weight.dtype]
    rotary_dim, max_pos = 0, 0
    if table is not None:
        _need(table.dim() == 2 and table.dtype == torch.float32, "table must be float32 (P, R)")
        max_pos, rotary_dim = table.shape
        _need(rotary_dim % 2 == 0 and rotary_dim <= D, "rotary dim must be even and at most D")
        _need(max_kv_len <= max_pos, "the step reaches position %d, the rotation table ends at %d"
              % (max_kv_len - 1, max_pos - 1))
    page, stride = 0, 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "a cache needs k, v and a block table")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == Hkv and k_cache.shape[3] == D
              and v_cache.shape == (k_cache.shape[0], Hkv, D, k_cache.shape[2])
              and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype,
              "caches must be keys (pages, Hkv, page, D) and values (pages, Hkv, D, page) of the activation dtype")
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 (B, W)")
        page, stride = k_cache.shape[2], block_table.shape[1]
    if T:
        _check(library("rotary").q3_qk_norm_rope_store(
            _ptr(qkv), _ptr(q_weight), _ptr(k_weight), w_dtype, ctypes.c_float(eps),
            _ptr(table), rotary_dim, max_pos, _ptr(positions), _ptr(seq_index),
            _ptr(block_table), stride, 0 if block_table is None else block_table.shape[0],
            _ptr(k_cache), _ptr(v_cache), page, 0 if k_cache is None else k_cache.shape[0],
            T, Hq, Hkv, D, _DT[qkv.dtype], _ptr(cu_seqlens_q), _ptr(kv_lens),
            0 if kv_lens is None else kv_lens.shape[0], int(max_q_len), int(max_kv_len), _stream()),
            "qk_norm_rope_store")
    return qkv


def paged_attention(q, num_q_heads, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens,
                    max_q_len, max_kv_len, scale, window=0, out=None, min_q_len=1, max_kv_len_of_many=None, softcap=0.0,
                    sink=None):
    """Causal softmax attention of packed query rows over paged keys and values.
    `softcap` > 0: a score s enters the softmax as softcap * tanh(s * scale / softcap); that form
    exists for the sizes the matrix cores take (a second build of the same kernels) and no other.
    `sink` float32 (Hq,): exp(sink[h]) joins the denominator of head h's softmax (no key, no value).

    q is (T, Hq, D) seen through a row stride (a view of the qkv buffer is
    fine). Keys are cached as (pages, Hkv, page, D), values as
    (pages, Hkv, D, page). Sequence b owns rows cu_seqlens_q[b]..cu_seqlens_q[b+1]; its keys
    0..kv_lens[b]-1 lie in pages block_table[b, j // page]; its query row i sits
    at position kv_lens[b] - q_len + i and sees keys at positions <= its own
    and, if window > 0, fewer than `window` behind it. Query head h reads
    key head h // (Hq / Hkv). Softmax statistics and accumulation are float32.
    `max_q_len` and `min_q_len` bound the sequences' row counts (they choose
    between the kernels for few and for many rows; loose bounds cost time only).
    `max_kv_len_of_many`: the most keys of a sequence that brings many rows, if
    the caller knows it (it decides whether such sequences' keys are shared out
    over several blocks; `max_kv_len` stands in).

    bfloat16 with head size 64 or 128 and a page size that is a power of two from 16
    runs on the matrix cores; everything else (float32, other head sizes in
    steps of 16 up to 256, other page sizes) takes the general kernel.
    """
    _dev(k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, out, sink)
    if sink is not None:
        _f32(sink, (num_q_heads,), "sink")
    _need(q.is_cuda and q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2],
          "q must be (T, Hq, D) with contiguous heads")
    T, Hq, D = q.shape
    _need(Hq == num_q_heads, "q's head count differs from num_q_heads")
    _need(q.dtype in _DT and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "q and the caches must share bfloat16 or float32")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == D, "the key cache must be (pages, Hkv, page, D)")
    Hkv, page = k_cache.shape[1], k_cache.shape[2]
    _need(v_cache.shape == (k_cache.shape[0], Hkv, D, page), "the value cache must be (pages, Hkv, D, page)")
    _need(Hq % Hkv == 0, "query heads must be a multiple of key heads")
    _need(D % 16 == 0 and 16 <= D <= 256, "head_dim must be a multiple of 16 in 16..256, found %d" % D)
    B = kv_lens.shape[0]
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.shape == (B + 1,), "cu_seqlens_q must be int32 (B+1,)")
    _need(kv_lens.dtype == torch.int32, "kv_lens must be int32 (B,)")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.shape[0] >= B,
          "block_table must be int32 (B, W)")
    _need(block_table.shape[1] * page >= max_kv_len, "block_table is narrower than the longest sequence")
    _need(1 <= min_q_len <= max_q_len, "need 1 <= min_q_len <= max_q_len")
    if out is None:
        out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, Hq * D) and out.dtype == q.dtype, "out must be (T, Hq D)")
    if T and B:
        lib = library("attention_capped" if softcap > 0 else "attention")
        if softcap > 0:
            _need(lib.q3_paged_attention_fast_path(Hq, Hkv, D, page, _DT[q.dtype]) and q.stride(0) % 8 == 0,
                  "capped scores need bfloat16, a head size of 64 or 128 and pages of a power of two from 16")
            lib.q3_set_score_cap.restype = None
            lib.q3_set_score_cap(ctypes.c_float(softcap))
        splits, workspace, prompt_splits, prompt_workspace = 1, None, 1, None
        if lib.q3_paged_attention_fast_path(Hq, Hkv, D, page, _DT[q.dtype]):
            if min_q_len * (Hq // Hkv) <= 16:
                splits = _splits(B, Hkv, max_kv_len)   # few rows per sequence: the keys go over several blocks
                if splits > 1:
                    lib.q3_paged_attention_workspace.restype = ctypes.c_long
                    n = lib.q3_paged_attention_workspace(B, Hkv, D, splits)
                    workspace = torch.empty((n,), dtype=torch.float32, device=q.device)
            if max_q_len * (Hq // Hkv) > 16:           # few long sequences over many keys: likewise
                longest = max_kv_len if max_kv_len_of_many is None else max_kv_len_of_many
                prompt_splits = lib.q3_paged_attention_prompt_splits(T, Hq, Hkv, int(longest))
                if prompt_splits > 1:
                    prompt_workspace = torch.empty((T * Hq * prompt_splits * (D + 2),), dtype=torch.float32,
                                                   device=q.device)
        _check(lib.q3_paged_attention(
            _ptr(q), q.stride(0), _ptr(out), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0],
            _ptr(block_table), block_table.shape[1], _ptr(cu_seqlens_q), _ptr(kv_lens),
            B, T, Hq, Hkv, D, page, ctypes.c_float(scale), int(window), int(max_q_len), int(min_q_len),
            int(max_kv_len), _DT[q.dtype], splits, _ptr(workspace), prompt_splits, _ptr(prompt_workspace), _ptr(sink),
            _stream()),
            "paged_attention")
    return out


def _splits(B, Hkv, max_kv_len):
    """Into how many blocks a sequence's keys are split when a step has few rows per sequence:
    until the chip is full, two blocks a compute unit and no more (the blocks beyond 512 run when
    the others have ended: 24 requests of 8 key heads over 768 keys take 27 us in two parts and 31
    in three, 12 requests over 2,000 keys 30 us in five parts and 35 in six); beyond 32 parts the
    merge costs more than the split gains. Two corrections to that, both measured with 8 key heads
    of 128: with 8,192 keys or more a block's work dwarfs its start and what counts is that the
    blocks come in even rounds, so at least eight parts are taken up to 384 (sequence, key head)
    pairs and four beyond (33 sequences over 8,200 keys: 257 us whole, 199 in eight parts; 40: 272
    and 232; 24: 156 in two parts, 143 in eight; 48: 295 whole, 274 in four; over 32,000 keys 955
    and 713, 1,022 and 832, 557 and 511, 1,110 and 1,018); and 257 to 320 pairs over fewer keys are
    split in three (33 sequences over 2,100 keys: 78 us whole, 70 in three; 40: 85 and 78; from 48
    sequences on one part is the fastest there)."""
    pairs = B * Hkv
    splits = max(1, min(max_kv_len // 64, 512 // pairs, 32))
    if max_kv_len >= 8192 and pairs < 512:
        splits = max(splits, 8 if pairs <= 384 else 4)
    elif 256 < pairs <= 320 and max_kv_len >= 1024:
        splits = 3
    return splits


def decode_attention_takes(num_q_heads, num_kv_heads, head_dim, page_size, dtype, rotary_dim=0):
    """Whether `decode_attention` serves these sizes (the caller then skips `qk_norm_rope_store`)."""
    if dtype != torch.bfloat16:
        return False
    return bool(library("attention").q3_decode_attention_takes(
        num_q_heads, num_kv_heads, head_dim, page_size, _DT[dtype], int(rotary_dim)))


def decode_attention(qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table, cu_seqlens_q,
                     kv_lens, max_kv_len, scale, window=0, q_weight=None, k_weight=None, eps=0.0, table=None,
                     store=True):
    """`qk_norm_rope_store` and `paged_attention` of a step in which every sequence brings one
    token, in one kernel: qkv (B, (Hq + 2 Hkv) D) bfloat16 holds the raw projections of
    sequence b's token in row b; the new key and value go to position kv_lens[b] - 1 of the
    caches (unless `store` is false: a layer that reads another layer's cache) and the
    attention output (B, Hq D) is returned. qkv is left as it was."""
    _dev(qkv, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, q_weight, k_weight, table)
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    B = kv_lens.shape[0]
    _need(qkv.dtype == torch.bfloat16 and qkv.shape == (B, (Hq + 2 * Hkv) * D), "qkv must be bfloat16 (B, (Hq + 2 Hkv) D)")
    _need(k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16 and k_cache.dim() == 4
          and k_cache.shape[1] == Hkv and k_cache.shape[3] == D, "key cache must be bfloat16 (pages, Hkv, page, D)")
    page = k_cache.shape[2]
    _need(v_cache.shape == (k_cache.shape[0], Hkv, D, page), "value cache must be (pages, Hkv, D, page)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= B, "block table int32 (B, blocks)")
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.shape == (B + 1,), "cu_seqlens_q int32 (B + 1,)")
    _need(kv_lens.dtype == torch.int32, "kv_lens int32 (B,)")
    _need((q_weight is None) == (k_weight is None), "q and k norm weights come together")
    w_dtype = 0
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype == k_weight.dtype
              and q_weight.dtype in _DT, "norm weights (D,) of one dtype")
        w_dtype = _DT[q_weight.dtype]
    rotary_dim = max_pos = 0
    if table is not None:
        _need(table.dtype == torch.float32 and table.dim() == 2, "rotation table float32 (positions, rotary_dim)")
        max_pos, rotary_dim = table.shape
        _need(max_kv_len <= max_pos, "the step reaches position %d, the rotation table ends at %d"
              % (max_kv_len - 1, max_pos - 1))
    _need(decode_attention_takes(Hq, Hkv, D, page, qkv.dtype, rotary_dim), "sizes the decoding kernel does not take")
    out = torch.empty((B, Hq * D), dtype=qkv.dtype, device=qkv.device)
    if B:
        lib = library("attention")
        splits, workspace = _splits(B, Hkv, max_kv_len), None
        if splits > 1:
            lib.q3_paged_attention_workspace.restype = ctypes.c_long
            workspace = torch.empty((lib.q3_paged_attention_workspace(B, Hkv, D, splits),), dtype=torch.float32,
                                    device=qkv.device)
        _check(lib.q3_decode_attention(
            _ptr(qkv), _ptr(out), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], _ptr(block_table),
            block_table.shape[1], _ptr(cu_seqlens_q), _ptr(kv_lens), B, Hq, Hkv, D, page, ctypes.c_float(scale),
            int(window), splits, _ptr(workspace), _ptr(q_weight), _ptr(k_weight), w_dtype, ctypes.c_float(eps),
            _ptr(table), int(rotary_dim), int(max_pos), 1 if store else 0, int(max_kv_len), _stream()),
            "decode_attention")
    return out


def tile_weight(weight):
    """A copy of a bfloat16 matrix (N, K) in the order the few-row product kernel reads it:
    [N / 16 slabs][K / 32 steps][64 lanes][8], lane = (n % 16) + 16 * ((k % 32) // 8), rows
    padded with zeros to a multiple of 16. None if the matrix is not bfloat16 or K is not a
    multiple of 32 (the row-major kernel then serves it)."""
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] % 32:
        return None
    N, K = weight.shape
    N16 = -(-N // 16) * 16
    if N16 != N:
        weight = torch.cat((weight, weight.new_zeros((N16 - N, K))), dim=0)
    tiles = weight.view(N16 // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4)   # slab, step, group, row, 8
    return tiles.contiguous().view(-1)


FEW_ROWS = 16                   # the few-row kernel's rows: one matrix instruction's worth of x
SMALL_WEIGHT_BYTES = 18 << 20   # up to this size the few-row kernel serves 32 rows, up to half of it 64


def few_rows_limit(weight):
    """Up to how many rows of x the few-row kernel serves a product with `weight` from its tiled
    copy: 16, or 32 or 64 for a small weight. The kernel works on 16 rows of x at a time; more
    rows are further sets of blocks that read the weight again. For a small weight that reading
    comes out of the caches and costs less than what the tiled kernel needs beyond 16 rows, a
    second kernel that adds its shares of K. Measured inside a graph, the product with its norm's
    work, few-row kernel against tiled kernel, in microseconds: 8 MB (4,096 x 1,024) at 24, 32, 48
    and 64 rows 5.8, 6.1, 8.4, 9.6 against 9.2, 9.6, 10.1, 10.9; 17 MB at 24, 32 and 48 rows 8.1,
    8.8, 11.9 against 9.9, 10.3, 11.5; 50 MB at 24 rows 20.0 against 15.0."""
    size = weight.numel() * weight.element_size()
    return FEW_ROWS * (4 if 2 * size <= SMALL_WEIGHT_BYTES else 2 if size <= SMALL_WEIGHT_BYTES else 1)


def sums_stride(M):
    """Columns of a tensor of rows' partial sums of squares for M rows (see `linear_residual_norm`)."""
    return -(-M // 16) * 16


def _tiled_ok(tiled, weight, M):
    if tiled is None or not 1 <= M <= few_rows_limit(weight):
        return False
    N, K = weight.shape
    _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous()
          and tiled.numel() == (-(-N // 16) * 16) * K and K % 32 == 0,
          "the tiled copy does not belong to this weight")
    return True


def _check_sums(sums, M):
    _dev(sums)
    _need(sums.dtype == torch.float32 and sums.dim() == 2 and sums.shape[1] == sums_stride(M) and sums.shape[0] > 0
          and sums.is_contiguous(), "row sums must be float32 (P, M rounded up to 16)")


def _row_sums_args(unscaled, M, K):
    """The few-row kernel's arguments for rows that still lack their 1 / rms factor: `unscaled` =
    (sums (P, M rounded up to 16) float32, eps, width) as `linear_residual_norm` leaves them."""
    if unscaled is None:
        return None, 0, ctypes.c_float(0.0), 0, 0
    sums, eps, width = unscaled
    _check_sums(sums, M)
    _need(width == K, "the rows' width must be the product's inner size")
    return _ptr(sums), sums.shape[0], ctypes.c_float(eps), int(width), sums.shape[1]


FUSED_ROWS_FEW, FUSED_ROWS_MOST = FEW_ROWS, 128


def fused_rows_take(weight, M):
    """Whether the tiled kernel carries a norm for `M` rows of a product with `weight` (N, K):
    more than 16 rows, at most 128 (beyond that the vendor library's products with the norms as
    kernels of their own are faster), bfloat16, K a multiple of 64 and N of 4. (Where the few-row
    kernel takes the rows too, a small weight's 17 to 32 or 64, that one is used.)"""
    return (FUSED_ROWS_FEW < M <= FUSED_ROWS_MOST and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] % 64 == 0 and weight.shape[0] % 4 == 0 and weight.is_contiguous())


def _tiles_scaled(x, weight, out, unscaled, swiglu, what):
    sums, eps, width = unscaled
    M, K = x.shape
    _check_sums(sums, M)
    _need(width == K, "the rows' width must be the product's inner size")
    _need(x.is_contiguous() and out.is_contiguous(), "operands must be contiguous")
    _check(_matmul().q3_tiles_scaled(
        _ptr(x), _ptr(weight), _ptr(out), M, weight.shape[0], K, _DT[out.dtype], 1 if swiglu else 0, _ptr(sums),
        sums.shape[0], sums.shape[1], ctypes.c_float(eps), int(width), _stream()), what)
    return out


STREAM_ROWS_MOST = 96


STREAM_ROWS_LEAST = 9      # of a gate/up product that runs whole; every other product from 17 rows


def stream_plan(M, N, K, swiglu=False):
    """How the weight-streaming kernel for 17 to 96 rows (9 to 96 of a gate/up product with the
    activation) would serve a product with a tile-ordered weight of (N, K) under the current
    settings: the slabs of 16 weight rows per block (6 or 4), or None where it leaves the product
    to the other kernels (small weights, slabs that do not fill the chip in one round of blocks,
    `matmul_kernels` other than "both", the tuner on)."""
    ws = _matmul().q3_stream_plan(int(M), int(N), int(K), 1 if swiglu else 0)
    return int(ws) if ws else None


def _stream_product(x, weight, tiled, out, swiglu, unscaled, what):
    """The product by the weight-streaming kernel, if it takes it: True if `out` is written."""
    M, K = x.shape
    N = weight.shape[0]
    least = STREAM_ROWS_LEAST if swiglu else FEW_ROWS + 1
    if tiled is None or not least <= M <= STREAM_ROWS_MOST or K % 32 or not x.is_contiguous() or not out.is_contiguous():
        return False
    _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous()
          and tiled.numel() == (-(-N // 16) * 16) * K, "the tiled copy does not belong to this weight")
    sums, chunks, stride, eps, width = None, 0, 0, 0.0, 0
    if unscaled is not None:
        sums, eps, width = unscaled
        _check_sums(sums, M)
        _need(width == K, "the rows' width must be the product's inner size")
        chunks, stride = sums.shape
    status = _matmul().q3_stream_product(
        _ptr(x), _ptr(tiled), _ptr(out), M, N, K, _DT[out.dtype], 1 if swiglu else 0, _ptr(sums), chunks, stride,
        ctypes.c_float(eps), int(width), _stream())
    if status == _DECLINED:
        return False
    _check(status, what)
    return True


def linear(x, weight, out_dtype=None, out=None, tiled=None, unscaled=None):
    """out = x @ weight^T with float32 accumulation. x (M, K), weight (N, K).
    `tiled` is `tile_weight(weight)`, if the caller keeps one: few rows are then served from it.
    `unscaled` (see `linear_residual_norm`) says that x's rows still lack their 1 / rms factor;
    the product's rows receive it. Only the few-row kernel on a tiled weight does this.

    float32 operands take a float32 kernel with no reduced-precision mode;
    bfloat16 operands with at most 16 rows (32 or 64 with the tiled copy of a small
    weight, `few_rows_limit`) take a weight-streaming matrix-core kernel; bfloat16 with
    more rows is the vendor library's product or the tiled kernel's.
    """
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    _need(x.dtype in _DT and weight.dtype == x.dtype, "x and weight must share bfloat16 or float32")
    M, K = x.shape
    N = weight.shape[0]
    out_dtype = out_dtype or x.dtype
    _need(out_dtype in _DT, "out dtype must be bfloat16 or float32")
    _need(not (x.dtype == torch.float32 and out_dtype != torch.float32), "float32 inputs give float32 output")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _need(out.shape == (M, N) and out.dtype == out_dtype, "out must be (M, N) of out_dtype")
    if M and x.dtype == torch.bfloat16 and _tiled_ok(tiled, weight, M):
        sums, sums_rows, eps, width, stride = _row_sums_args(unscaled, M, K)
        _check(library("gemm").q3_linear_tiled(
            _ptr(x), _ptr(tiled), _ptr(out), M, N, K, _DT[out_dtype], 0, sums, sums_rows, eps, width,
            None, None, 0, None, stride, _stream()), "linear")
        return out
    if M and x.dtype == torch.bfloat16 and (unscaled is None or fused_rows_take(weight, M)) \
            and _stream_product(x, weight, tiled, out, False, unscaled, "linear"):
        return out
    if unscaled is not None and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        return _tiles_scaled(x, weight, out, unscaled, False, "linear")
    _need(unscaled is None, "unscaled rows need bfloat16 and few rows with a tiled weight (few_rows_limit), or 17 to "
          "128 rows with an inner size that is a multiple of 64")
    if M and x.dtype == torch.bfloat16 and not library("gemm").q3_linear_is_skinny(M, N, K, 1):
        # bfloat16 products with many rows go to the vendor library (hipBLASLt), as the
        # reference's engine uses its vendor library for them, or to the hand-written tiled
        # kernel, as a table of sizes and a rule of thumb say; accumulation is float32.
        # Few rows take the weight-streaming kernel below.
        _need(x.is_contiguous() and weight.is_contiguous() and out.is_contiguous(), "operands must be contiguous")
        status = _matmul().q3_matmul(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[out_dtype], _stream())
        if status == _UNSUPPORTED:
            # a size neither hipBLASLt nor the tiled kernel has a kernel for (an odd inner size,
            # say): plain multiply-adds with float32 sums
            linear_plain(x, weight, out)
        else:
            _check(status, "matmul")
    elif M:
        _check(library("gemm").q3_linear(
            _ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _DT[out_dtype], _stream()), "linear")
    return out


def linear_plain(x, weight, out):
    """out = x @ weight^T by plain multiply-adds with float32 sums, for any size: what serves a
    bfloat16 product with more than 16 rows that neither the vendor library nor the tiled
    kernel takes, and every float32 product."""
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1] and x.dtype in _DT
          and weight.dtype == x.dtype, "x (M, K) and weight (N, K) of one dtype")
    M, K = x.shape
    N = weight.shape[0]
    _need(out.shape == (M, N) and out.dtype in _DT and not (x.dtype == torch.float32 and out.dtype != torch.float32),
          "out must be (M, N); float32 inputs give float32 output")
    lib = library("gemm")
    _need(M > 16 or x.dtype == torch.float32 or not lib.q3_linear_is_skinny(M, N, K, 1),
          "bfloat16 products of up to 16 rows are the weight-streaming kernel's")
    if M:
        _check(lib.q3_linear(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _DT[out.dtype], _stream()),
               "linear_plain")
    return out


def linear_swiglu(x, weight, tiled=None, unscaled=None):
    """swiglu(x @ weight^T) for a weight whose rows interleave gate and up (row 2i gate's, row
    2i + 1 up's): (M, K) x (2I, K) -> (M, I). With few bfloat16 rows the activation is the
    product kernel's epilogue; otherwise it is the product followed by `swiglu`.
    `unscaled`: as for `linear`."""
    _dev(x, weight)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1] and weight.shape[0] % 2 == 0,
          "x (M, K) and weight (2I, K)")
    _need(x.dtype in _DT and weight.dtype == x.dtype, "x and weight must share bfloat16 or float32")
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype == torch.bfloat16 and tiled is not None and STREAM_ROWS_LEAST <= M <= FEW_ROWS and N % 4 == 0:
        # a whole gate/up product of 9 to 16 rows: the streaming kernel, where it takes the size
        if unscaled is not None:
            _need(unscaled[0].dim() == 2 and unscaled[0].shape[1] == sums_stride(M), "row sums (P, M rounded up to 16)")
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if _stream_product(x, weight, tiled, out, True, unscaled, "linear_swiglu"):
            return out
    if M and x.dtype == torch.bfloat16 and _tiled_ok(tiled, weight, M):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        sums, sums_rows, eps, width, stride = _row_sums_args(unscaled, M, K)
        _check(library("gemm").q3_linear_tiled(
            _ptr(x), _ptr(tiled), _ptr(out), M, N, K, 1, 1, sums, sums_rows, eps, width,
            None, None, 0, None, stride, _stream()), "linear_swiglu")
        return out
    if M and x.dtype == torch.bfloat16 and tiled is not None and FEW_ROWS < M <= STREAM_ROWS_MOST \
            and (unscaled is None or fused_rows_take(weight, M)):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if _stream_product(x, weight, tiled, out, True, unscaled, "linear_swiglu"):
            return out
    if unscaled is not None and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        return _tiles_scaled(x, weight, out, unscaled, True, "linear_swiglu")
    _need(unscaled is None, "unscaled rows need bfloat16 and few rows with a tiled weight (few_rows_limit), or 17 to "
          "128 rows with an inner size that is a multiple of 64")
    if M and library("gemm").q3_linear_is_skinny(M, N, K, _DT[x.dtype]):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        _check(library("gemm").q3_linear_swiglu(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _stream()),
               "linear_swiglu")
        return out
    return swiglu(linear(x, weight, tiled=tiled))


def linear_residual_norm(x, weight, tiled, residual, norm_weight):
    """residual += x @ weight^T, and the next norm's input prepared in the same kernel.

    x (M, K) bfloat16, weight (N, K); residual (M, N) float32 is updated in place (the product
    is rounded to bfloat16 before the addition, as a product written out and added by the norm
    kernel would be). Returns (values, sums): values (M, N) bfloat16 = residual * norm_weight,
    and sums (P, M rounded up to 16) float32, the rows' sums of squares of the new residual in P
    partial sums (row m of the stream in column m). The norm's result is
    values * rsqrt(sum / N + eps) row by row; `linear` and `linear_swiglu` apply that factor to
    their products when given `unscaled=(sums, eps, N)`.

    Up to `few_rows_limit(weight)` rows, with the weight's tiled copy and N a multiple of 16, it
    is the few-row kernel's epilogue (P = N / 16, partial sums of 16 columns). With more rows, up
    to 128 (`fused_rows_take`; `tiled` is not used), the tiled kernel's partial products are added
    by a second kernel that does the same (P = ceil(N / 1024)). There the result is None, and
    nothing was done, for a size at which the plain product (`linear`) followed by the norm's own
    kernel is the faster way."""
    _dev(x, weight, tiled, residual, norm_weight)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    M, K = x.shape
    N = weight.shape[0]
    _need(residual.shape == (M, N) and residual.dtype == torch.float32 and residual.is_contiguous(),
          "residual must be float32 (M, N)")
    _need(norm_weight.shape == (N,) and norm_weight.dtype in _DT and norm_weight.is_contiguous(), "norm weight (N,)")
    values = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    few = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and N % 16 == 0 and _tiled_ok(tiled, weight, M)
    if not few and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        _need(x.is_contiguous(), "x must be contiguous")
        lib = _matmul()
        sums = torch.empty((lib.q3_tiles_residual_chunks(N), sums_stride(M)), dtype=torch.float32, device=x.device)
        status = lib.q3_tiles_residual(
            _ptr(x), _ptr(weight), M, N, K, _ptr(residual), _ptr(norm_weight), _DT[norm_weight.dtype], _ptr(values),
            _ptr(sums), sums.shape[1], _stream())
        if status == _DECLINED:
            return None
        _check(status, "linear_residual_norm")
        return values, sums
    _need(few, "bfloat16, a tiled weight with a width that is a multiple of 16 and no more rows than few_rows_limit, "
          "or 17 to 128 rows with an inner size that is a multiple of 64")
    sums = torch.empty((N // 16, sums_stride(M)), dtype=torch.float32, device=x.device)
    _check(library("gemm").q3_linear_tiled(
        _ptr(x), _ptr(tiled), _ptr(values), M, N, K, 1, 2, None, 0, ctypes.c_float(0.0), 0,
        _ptr(residual), _ptr(norm_weight), _DT[norm_weight.dtype], _ptr(sums), sums.shape[1], _stream()),
        "linear_residual_norm")
    return values, sums


def sample(logits, temperature, top_k, seed, counter, out=None, any_top_k=True):
    """One token per row of float32 logits (R, V).

    Row r: temperature[r] <= 0 takes the arg-max (lowest index among equals).
    Otherwise it draws from softmax(logits / temperature) restricted, when
    top_k[r] > 0, to logits not below the k-th largest; the draw is the
    arg-max of logits / temperature + Gumbel noise from a counter-based
    generator keyed by (seed[r], counter[r], column), so a request's tokens do
    not depend on what else is in the batch. `any_top_k=False` promises that no row has a
    top_k in effect, which saves the selection pass.
    """
    _dev(logits, temperature, top_k, seed, counter, out)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "logits must be float32 (R, V)")
    R, V = logits.shape
    _need(temperature.shape == (R,) and temperature.dtype == torch.float32, "temperature float32 (R,)")
    _need(top_k.shape == (R,) and top_k.dtype == torch.int32, "top_k int32 (R,)")
    _need(seed.shape == (R,) and seed.dtype == torch.int64, "seed int64 (R,)")
    _need(counter.shape == (R,) and counter.dtype == torch.int32, "counter int32 (R,)")
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out.shape == (R,) and out.dtype == torch.int32, "out int32 (R,)")
    if R:
        lib = library("sampling")
        lib.q3_sample_workspace.restype = ctypes.c_long
        workspace = torch.empty((lib.q3_sample_workspace(R, V) + 7) // 8, dtype=torch.int64, device=logits.device)
        _check(lib.q3_sample(
            _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(seed), _ptr(counter), _ptr(out),
            R, V, 1 if any_top_k else 0, _ptr(workspace), _stream()), "sample")
    return out


def measured_read_rate(gigabytes=4.0, repeats=5):
    """Bytes per second at which a kernel reads a buffer of `gigabytes` that no cache holds (the
    fastest of `repeats` passes): what this GPU's memory delivers to a long, plain read."""
    lib = library("probes")
    count = int(gigabytes * 1e9) // 16 * 16
    buffer = torch.zeros(count, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    best = 0.0
    for blocks in (2048, 4096, 8192):
        for _ in range(repeats):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            _check(lib.q3_probe_read(_ptr(buffer), ctypes.c_size_t(count), _ptr(sink), blocks, _stream()), "probe_read")
            end.record()
            end.synchronize()
            best = max(best, count / (begin.elapsed_time(end) * 1e-3))
    return best


def measured_matrix_rate(repeats=5, shape=None, blocks=256 * 8, iters=4096):
    """Floating-point operations per second of the bfloat16 matrix instructions with their
    operands in registers, all compute units busy: the better of v_mfma_f32_16x16x32_bf16 and
    v_mfma_f32_32x32x16_bf16 (`shape` 0 or 1 asks for one of them)."""
    lib = library("probes")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    best = 0.0
    for which in ((0, 1) if shape is None else (shape,)):
        for _ in range(repeats):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            _check(lib.q3_probe_mfma(int(blocks), int(iters), which, _ptr(sink), ctypes.byref(flops), _stream()),
                   "probe_mfma")
            end.record()
            end.synchronize()
            best = max(best, flops.value / (begin.elapsed_time(end) * 1e-3))
    return best
