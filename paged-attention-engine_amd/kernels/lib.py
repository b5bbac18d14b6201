"""ctypes bindings of the gfx950 kernel library and thin, checked wrappers.

Every wrapper takes torch tensors that already live on the GPU, checks on the
host that shapes and dtypes match what the kernel and its grid assume, launches
on torch's current stream and raises `KernelError` with the library's message
on refusal.  There is no fallback: without the library or without a GPU these
functions raise.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from typing import Optional

import torch

from .build import ensure_built

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_lib = None


def library():
    """The loaded kernel library (built at the first call if necessary)."""
    global _lib
    if _lib is None:
        # PAE_KERNEL_LIBRARY: a library built by hand from the same sources (a variant under measurement)
        path = os.environ.get("PAE_KERNEL_LIBRARY") or ensure_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as err:
            raise KernelError(f"cannot load the kernel library {path}: {err}") from err
        _declare(lib)
        _lib = lib
    return _lib


def loaded_library_path() -> Optional[str]:
    return getattr(_lib, "_name", None) if _lib is not None else None


def _declare(lib) -> None:
    lib.pae_last_error.restype = c_char_p
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sig = {
        "pae_device_arch": [c_char_p, I],
        "pae_embedding": [I, P, P, P, I, I, I, F, P],
        "pae_logits_finish": [P, L, F, F, P],
        "pae_add_rmsnorm": [I, P, P, I, L, P, I, F, P, P, I, I, I, P],
        "pae_residual_add": [I, P, P, L, P],
        "pae_scatter_i32": [P, P, P, P, I, P],
        "pae_copy_i32": [P, P, I, P],
        "pae_rope_table": [P, P, P, I, I, P],
        "pae_rope_kv_write": [I, P, L, I, I, I, I, I, P, I, P, P, P, P, I, I, P, P, I, P],
        "pae_swiglu": [I, P, P, I, I, I, P],
        "pae_gemm_skinny": [I, P, L, P, L, P, P, I, I, I, I, I, L, P, P, P, I, F, P, L, P, I, P, P],
        "pae_gemm_skinny_rope": [P, L, P, L, P, P, I, I, I, I, I, I, I, P, P, P, P, I, I, P, P, I, P, P, P, I, F, P],
        "pae_embedding_rows": [I, P, P, P, I, I, I, F, P, P, I, P, P],
        "pae_scaled_rows": [P, P, P, I, F, I, I, P],
        "pae_skinny_ticket_slots": [I, I],
        "pae_gemm_skinny_act": [P, L, P, L, P, P, I, I, I, I, I, P, P, I, P],
        "pae_gemm_plain": [I, I, P, L, P, L, P, P, I, I, I, I, P],
        "pae_gemm_skinny_gated": [P, L, P, L, P, I, I, I, I, P, P, I, P],
        "pae_paged_attention_generic": [I, P, L, P, L, P, P, P, P, P, I, I, I, I, I, I, F, I, P],
        "pae_paged_attention_capped": [I, P, L, P, L, P, P, P, P, P, I, I, I, I, I, I, I, F, I, F, P, P],
        "pae_qk_norm_rotate_store": [I, P, L, I, I, I, I, I, P, P, I, F, I, I, P, F, P, P, P, I, I, P, P, I, I, P],
        "pae_paged_attention_masked": [I, P, L, P, L, P, P, P, P, P, I, I, I, I, I, I, I, F, I, F, P, I, P, P, L, I, P],
        "pae_hyper_norm": [I, P, I, P, I, L, P, I, P, P, P, P, I, F, P, P, I, I, I, P],
        "pae_hyper_spread": [P, P, I, I, I, P],
        "pae_hyper_collapse": [P, P, I, I, I, P],
        "pae_conv_norm_store": [I, P, L, P, L, I, I, P, P, P, P, P, P, L, I, I, I, I, I, I, F, P, I, I, P, P, P],
        "pae_latent_prepare": [I, P, L, P, L, I, I, I, I, I, I, I, P, I, F, P, P, P, P, I, I, P, P, P],
        "pae_heads_product_few": [P, L, L, P, L, L, P, I, I, I, I, P],
        "pae_latent_attn_supported": [I, I, I],
        "pae_latent_attn_columns": [I, I],
        "pae_latent_attn_bf16": [P, L, P, L, P, P, P, I, I, P, P, I, I, I, I, I, F, I, I, P, P, P, P],
        "pae_latent_attn_split": [],
        "pae_gated_act": [I, P, P, I, I, I, I, P],
        "pae_gemm_plain_batched": [I, I, P, L, L, P, L, L, P, L, P, I, I, I, I, I, P],
        "pae_rows_from_residual": [I, P, P, L, P],
        "pae_norm_scale_add": [I, P, P, I, L, P, I, F, F, P, I, I, P],
        "pae_activation": [I, P, L, I, P],
        "pae_delta_rule_step": [I, P, L, I, I, P, P, P, P, P, P, L, I, I, I, I, I, P, P, F, P, L, P, I, F, P, P,
                                P, L, I, P, L, P, L, I, P],
        "pae_matrix_memory_step": [I, P, L, P, L, P, I, I, P, P, I, I, I, F, P, L, P, L, P, I, F, F, P, P, P],
        "pae_embedding_pairs": [I, P, P, P, P, P, P, P, P, I, I, I, F, I, I, I, P],
        "pae_sum_norm2": [I, P, I, P, P, P, P, P, P, I, P, I, F, P, P, P, I, I, I, P],
        "pae_project_f32": [I, P, L, P, L, P, P, I, I, I, I, P],
        "pae_moe_route": [P, I, I, I, I, I, F, P, P, P, P],
        "pae_norm_join": [I, P, I, P, P, P, P, P, P, I, F, P, I, F, P, P, I, I, P],
        "pae_linear_attention_step": [I, P, L, P, L, P, I, F, P, L, I, I, I, P, P, I, I, I, P, L, P, I, F, P, P, P],
        "pae_embedding_positions": [I, P, P, P, P, P, I, I, I, F, P],
        "pae_token_gate": [I, P, P, L, P, P, I, I, I, P],
        "pae_moe_gate_up": [I, P, P, L, P, P, P, I, I, I, I, I, P],
        "pae_moe_down": [I, P, P, P, P, P, I, I, I, I, P],
        "pae_moe_tile_rows": [I],
        "pae_moe_max_tiles": [I, I],
        "pae_moe_tiles_supported": [I, I],
        "pae_moe_experts_tiles": [P, P, L, P, P, P, P, P, I, I, I, I, I, I, P, P, P, P],
        "pae_sample": [P, P, L, P, P, I, I, P, P, P, P],
        "pae_sample_chunks": [I],
        "pae_sample_static": [P, P, L, P, P, I, I, P],
        "pae_sample_static_slots": [],
        "pae_sample_static_prepare": [],
        "pae_attn_decode_bf16": [P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, P, P, P],
        "pae_attn_decode_split": [],
        "pae_attn_decode_biased_bf16": [P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, I, P, P, L, P, P, P],
        "pae_attn_prefill_biased_bf16": [P, L, P, L, P, P, P, I, P, P, I, I, I, I, I, F, I, I, P, P, L, P],
        "pae_attn_decode_capped_bf16": [P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, F, P, P, P, P],
        "pae_attn_prefill_capped_bf16": [P, L, P, L, P, P, P, I, P, P, I, I, I, I, I, F, I, F, P, P],
        "pae_attn_prefill_bf16": [P, L, P, L, P, P, P, I, P, P, I, I, I, I, I, F, I, P],
        "pae_program_phase_bytes": [],
        "pae_program_barrier_bytes": [],
        "pae_program_max_rows": [],
        "pae_program_max_groups": [],
        "pae_program_put_product": [P, I, I, P, L, P, L, P, P, I, I, I, I, I, P, P, P, I, F, P, L, P, I, P, P],
        "pae_program_put_product_rope": [P, I, P, L, P, L, P, P, I, I, I, I, I, I, I, P, P, P, P, I, I, P, P, I, P, P, P,
                                         I, F],
        "pae_program_put_attention": [P, I, P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, P, P],
        "pae_program_run": [P, I, P, P, I, I, I, I, P, P],
        "pae_program_activation_bytes": [I, I, I],
        "pae_program_lds_limit": [],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.pae_skinny_ticket_floats.argtypes = [I, I, I]
    lib.pae_skinny_ticket_floats.restype = c_int64
    lib.pae_delta_rule_work_floats.argtypes = [I, I, I, I, I, I]
    lib.pae_delta_rule_work_floats.restype = c_int64
    lib.pae_matrix_memory_work_floats.argtypes = [I, I, I, I]
    lib.pae_matrix_memory_work_floats.restype = c_int64
    lib.pae_linear_attention_work_floats.argtypes = [I, I, I, I]
    lib.pae_linear_attention_work_floats.restype = c_int64


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().pae_last_error().decode("utf-8", "replace"))


def _stream() -> int:
    # the raw handle of torch's current stream (also the capture stream while a graph records)
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def code_of(dtype: torch.dtype) -> int:
    try:
        return _CODE[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not one the kernels take (float32, bfloat16)") from None


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _param(t: Optional[torch.Tensor]):
    """(pointer, is_f32) of a vector parameter stored in float32 or bfloat16."""
    if t is None:
        return None, 0
    if t.dtype not in _CODE:
        raise KernelError(f"parameter dtype {t.dtype} not supported")
    return t.data_ptr(), 1 if t.dtype == torch.float32 else 0


def _check_pools(k_cache, v_cache, nkv: int, bs: int, hd: int) -> None:
    """Keys [block][kv head][bs][hd]; values transposed within the page, [block][kv head][hd][bs]."""
    assert tuple(k_cache.shape[1:]) == (nkv, bs, hd) and k_cache.is_contiguous()
    assert tuple(v_cache.shape) == (k_cache.shape[0], nkv, hd, bs) and v_cache.is_contiguous()
    assert k_cache.dtype == v_cache.dtype


def device_arch() -> str:
    buf = ctypes.create_string_buffer(64)
    _check(library().pae_device_arch(buf, 64))
    return buf.value.decode().split(":")[0]


def embedding(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = scale * table[ids[t]] as float32; ids int32 (checked against the table by the caller)."""
    _not_while_recording("embedding")
    _gpu(out, table, ids)
    T, H = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous()
    assert ids.dtype == torch.int32 and ids.numel() == T and table.shape[1] == H
    _check(library().pae_embedding(code_of(table.dtype), out.data_ptr(), table.data_ptr(), ids.data_ptr(),
                                   T, H, table.shape[0], float(scale), _stream()))


def embedding_positions(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, rows: torch.Tensor,
                        positions: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = scale * table[ids[t]] + rows[positions[t]] as float32: `rows` [max positions, H] holds a learned row
    per position, added unscaled.  The caller vouches that every position lies within `rows`."""
    _not_while_recording("embedding_positions")
    _gpu(out, table, ids, rows, positions)
    T, H = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous() and rows.is_contiguous()
    assert table.dtype == rows.dtype and table.shape[1] == H == rows.shape[1]
    for t in (ids, positions):
        assert t.dtype == torch.int32 and t.numel() == T and t.is_contiguous()
    _check(library().pae_embedding_positions(code_of(table.dtype), out.data_ptr(), table.data_ptr(), ids.data_ptr(),
                                             rows.data_ptr(), positions.data_ptr(), T, H, table.shape[0], float(scale),
                                             _stream()))


def token_gate(gate: torch.Tensor, columns: torch.Tensor, ids: torch.Tensor, kind: str) -> torch.Tensor:
    """[T, dim] in gate's type: act(gate[t]) * columns[ids[t]], `gate` [T, dim] a narrow product of the stream (a view
    of wider rows will do), `columns` [vocab, dim] a layer's columns of a second token table; float32 inside."""
    _not_while_recording("token_gate")
    _gpu(gate, columns, ids)
    T, dim = gate.shape
    assert gate.stride(1) == 1 and columns.is_contiguous() and columns.shape[1] == dim and columns.dtype == gate.dtype
    assert ids.dtype == torch.int32 and ids.numel() == T and ids.is_contiguous() and kind in ACTIVATIONS
    out = torch.empty((T, dim), dtype=gate.dtype, device=gate.device)
    _check(library().pae_token_gate(code_of(gate.dtype), out.data_ptr(), gate.data_ptr(), gate.stride(0), columns.data_ptr(),
                                    ids.data_ptr(), T, dim, ACTIVATIONS[kind], _stream()))
    return out


def logits_finish(logits: torch.Tensor, scale: float = 1.0, softcap: float = 0.0) -> None:
    """In place: logits = scale * logits, then with a soft cap c > 0, c * tanh(logits / c)."""
    _not_while_recording("logits_finish")
    _gpu(logits)
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    _check(library().pae_logits_finish(logits.data_ptr(), logits.numel(), float(scale), float(softcap), _stream()))


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None, write_residual: bool = True) -> None:
    """residual (+= delta); out = weight * round(residual * rsqrt(mean(residual^2) + eps)).

    `delta` is the pending branch output: [T, H] in out's dtype, or float32 partial sums
    [P, T, H] that are added in order.  With `rows` (int32), out[b] comes from source row
    rows[b] and nothing is written back."""
    _not_while_recording("add_rmsnorm")
    _gpu(residual, delta, weight, out, rows)
    H = residual.shape[-1]
    n = out.shape[0]
    assert residual.dtype == torch.float32 and residual.is_contiguous() and out.is_contiguous()
    assert out.shape[-1] == H and weight.numel() == H
    parts, part_stride = 0, 0
    if delta is not None:
        assert delta.is_contiguous()
        if delta.dim() == 3:
            assert delta.dtype == torch.float32 and delta.shape[1:] == residual.shape
            parts, part_stride = delta.shape[0], residual.numel()
        else:
            assert delta.dtype == out.dtype and delta.shape == residual.shape
    if rows is None:
        assert residual.shape[0] == n
    else:
        assert rows.dtype == torch.int32 and rows.numel() == n
        write_residual = False
    wp, wf = _param(weight)
    _check(library().pae_add_rmsnorm(code_of(out.dtype), residual.data_ptr(), _ptr(delta), parts, part_stride,
                                     wp, wf, float(eps),
                                     _ptr(rows), out.data_ptr(), n, H, 1 if write_residual else 0, _stream()))


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> None:
    _not_while_recording("residual_add")
    _gpu(residual, delta)
    assert residual.dtype == torch.float32 and residual.shape == delta.shape
    assert residual.is_contiguous() and delta.is_contiguous()
    _check(library().pae_residual_add(code_of(delta.dtype), residual.data_ptr(), delta.data_ptr(),
                                      residual.numel(), _stream()))


def copy_int32_from_pinned(dst: torch.Tensor, src: torch.Tensor, n: int) -> None:
    """dst[:n] = src[:n] by a kernel on the current stream; `src` is pinned host memory (which the
    GPU reads in place) and must stay as it is until the kernel has run."""
    _not_while_recording("copy_int32_from_pinned")
    _gpu(dst)
    assert dst.dtype == torch.int32 == src.dtype and dst.is_contiguous() and src.is_contiguous()
    assert src.is_pinned() and 0 <= n <= min(dst.numel(), src.numel())
    _check(library().pae_copy_i32(dst.data_ptr(), src.data_ptr(), n, _stream()))


def scatter_int32(dst: torch.Tensor, dst_idx: torch.Tensor, src: torch.Tensor, src_idx: torch.Tensor, n: int) -> None:
    """dst[dst_idx[i]] = src[src_idx[i]] for i < n (int32 everywhere; the index lists may be longer than n).
    The caller vouches for the indices: they are not checked on the device."""
    _not_while_recording("scatter_int32")
    _gpu(dst, dst_idx, src, src_idx)
    for t in (dst, dst_idx, src, src_idx):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert 0 <= n <= min(dst_idx.numel(), src_idx.numel())
    _check(library().pae_scatter_i32(dst.data_ptr(), dst_idx.data_ptr(), src.data_ptr(), src_idx.data_ptr(), n,
                                     _stream()))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """[T, len(inv_freq), 2] float32: cosine and sine of positions[t] * inv_freq[i]."""
    _gpu(positions, inv_freq)
    assert positions.dtype == torch.int32 and inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
    T, half = positions.numel(), inv_freq.numel()
    out = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
    _check(library().pae_rope_table(out.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half, _stream()))
    return out


def _check_cos_sin(cos_sin: Optional[torch.Tensor], rot: int, T: int) -> None:
    if rot:
        assert cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
        assert tuple(cos_sin.shape) == (T, rot // 2, 2)


def rope_kv_write(qkv: torch.Tensor, nh: int, nkv: int, hd: int, rot: int, cos_sin: Optional[torch.Tensor],
                  positions: torch.Tensor, tok_seq: Optional[torch.Tensor], block_tables: Optional[torch.Tensor],
                  block_size: int, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  bias: Optional[torch.Tensor] = None) -> None:
    """Rotate the query heads of `qkv` in place by the angles whose cosines and sines `cos_sin`
    holds ([T, rot / 2, 2], see `rope_table`); rotate the key heads and copy the value heads
    into their cache slots (skipped when `k_cache` is None: then the row holds query heads only
    and nkv must be 0).  With `bias` (one value per feature of the row) the row stands for the
    projection without its bias, which is added here first."""
    _not_while_recording("rope_kv_write")
    _gpu(qkv, cos_sin, positions, tok_seq, block_tables, k_cache, v_cache, bias)
    if bias is not None:
        assert bias.numel() == (nh + 2 * nkv) * hd
    T = qkv.shape[0]
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and positions.dtype == torch.int32 and positions.numel() == T
    write = k_cache is not None
    _check_cos_sin(cos_sin, rot, T)
    max_blocks = 0
    if write:
        assert v_cache is not None and k_cache.dtype == qkv.dtype == v_cache.dtype
        assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        _check_pools(k_cache, v_cache, nkv, block_size, hd)
        max_blocks = block_tables.shape[1]
    bp, bf = _param(bias)
    _check(library().pae_rope_kv_write(code_of(qkv.dtype), qkv.data_ptr(), qkv.stride(0), T, nh, nkv, hd, rot,
                                       bp, bf, _ptr(cos_sin) if rot else None, positions.data_ptr(), _ptr(tok_seq),
                                       _ptr(block_tables), max_blocks, block_size, _ptr(k_cache), _ptr(v_cache),
                                       1 if write else 0, _stream()))


def rotate_heads(x: torch.Tensor, num_heads: int, hd: int, rot: int, cos_sin: torch.Tensor,
                 positions: torch.Tensor) -> None:
    """Rotate the first `num_heads` heads (each `hd` wide) of every row of `x` in place; nothing is stored."""
    rope_kv_write(x, num_heads, 0, hd, rot, cos_sin, positions, None, None, 1, None, None)


def kv_store(qkv: torch.Tensor, nh: int, nkv: int, hd: int, positions: torch.Tensor, tok_seq: torch.Tensor,
             block_tables: torch.Tensor, block_size: int, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """Copy the key and value heads of rows [q heads | k heads | v heads] into their cache slots, as they are."""
    rope_kv_write(qkv, nh, nkv, hd, 0, None, positions, tok_seq, block_tables, block_size, k_cache, v_cache)


def swiglu(out: torch.Tensor, x: torch.Tensor, block: int = 0) -> None:
    """out[t, j] = silu(gate_j) * up_j for x of width 2 I: gate = x[:, :I], up = x[:, I:], or,
    with `block` > 0, blocks of `block` gate features each followed by their up features."""
    _not_while_recording("swiglu")
    _gpu(out, x)
    T, I = out.shape
    assert x.shape == (T, 2 * I) and x.dtype == out.dtype and x.is_contiguous() and out.is_contiguous()
    _check(library().pae_swiglu(code_of(x.dtype), out.data_ptr(), x.data_ptr(), T, I, block, _stream()))


def gated_act(out: torch.Tensor, x: torch.Tensor, kind: str, block: int = 0) -> None:
    """`swiglu` with the gate's activation by name (see ACTIVATIONS): out = act(gate) * up."""
    _not_while_recording("gated_act")
    _gpu(out, x)
    T, I = out.shape
    assert x.shape == (T, 2 * I) and x.dtype == out.dtype and x.is_contiguous() and out.is_contiguous()
    assert kind in ACTIVATIONS
    _check(library().pae_gated_act(code_of(x.dtype), out.data_ptr(), x.data_ptr(), T, I, block, ACTIVATIONS[kind],
                                   _stream()))


# ---------------------------------------------------------------------------------- decode programs
# A decode step's products and attention as one resident kernel (csrc/decode_program.hip).  While a
# program is recording, `gemm_skinny`, `gemm_skinny_rope` and `attn_decode` append a phase to it
# instead of launching; `rope_table`, which reads the step's positions only, runs at once; every other
# wrapper refuses.  `launch()` then runs the phases in the order they were recorded, each after the
# one before it has finished everywhere, as the separate launches would.
_RECORDING = None
PROGRAM_SPIN_LIMIT = 2_000_000  # polls of a barrier before a workgroup gives up (about two seconds)


def _not_while_recording(name: str) -> None:
    if _RECORDING is not None:
        raise KernelError(f"{name} cannot be a phase of a decode program; a part that calls it must not say it is fusable")


def program_max_rows() -> int:
    return library().pae_program_max_rows()


def program_takes_product(rows: int, K: int, splits: int, quad_bytes: int = 27 * 1024) -> bool:
    """Whether a decode program has the LDS for a product of `rows` rows over k ranges of K / splits
    (a workgroup keeps one range's activations there, beside its quads' own `quad_bytes` each)."""
    lib = library()
    return 2 * quad_bytes + lib.pae_program_activation_bytes(rows, K, splits) <= lib.pae_program_lds_limit()


_PROGRAM_BARRIERS: dict = {}  # (device index, workgroups) -> zeroed barrier block


class DecodeProgram:
    """Room for a list of phases (in pinned host memory, where it is written, and on the device, where
    the kernel reads it) and what running them needs.  A program recorded into a HIP graph keeps its
    list for as long as the graph lives: every replay copies it to the device again."""

    def __init__(self, device, max_phases: int, groups: Optional[int] = None) -> None:
        lib = library()
        self.device = torch.device(device)
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("a decode program's buffers must exist before a graph is recorded")
        with torch.cuda.device(self.device):
            most = lib.pae_program_max_groups()
        if most < 1:
            _check(most)
        self.groups = most if groups is None else int(groups)
        if not 1 <= self.groups <= most:
            raise KernelError(f"{self.groups} workgroups cannot all be resident (at most {most})")
        self.phase_bytes = lib.pae_program_phase_bytes()
        self.max_phases = max_phases
        ints = self.phase_bytes * max_phases // 4
        self.host = torch.zeros(ints, dtype=torch.int32, pin_memory=True)
        self.on_device = torch.zeros(ints, dtype=torch.int32, device=self.device)
        self.error = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        key = (self.device.index or 0, self.groups)
        if key not in _PROGRAM_BARRIERS:
            _PROGRAM_BARRIERS[key] = torch.zeros(lib.pae_program_barrier_bytes() // 4, dtype=torch.int32, device=self.device)
        self.barrier = _PROGRAM_BARRIERS[key]
        skinny_tickets(self.device)
        self.host_ptr = self.host.data_ptr()
        self.count = 0
        self.quad_lds = 0        # bytes of LDS a quad needs: the most any phase asked for
        self.activation_lds = 0  # bytes of LDS for a product's activations: likewise
        self.keep: list = []
        self._read: Optional[torch.cuda.Event] = None
        self.trace: Optional[torch.Tensor] = None  # int64 [phases, workgroups, 2] clock readings of the next launches, if set

    def begin(self) -> None:
        if self._read is not None:
            self._read.synchronize()  # the launch before has copied the list to the device
        self.count, self.quad_lds, self.activation_lds, self.keep = 0, 0, 0, []

    def room(self, phases: int) -> None:
        """Raise unless `phases` more fit the list (asked before a pae_program_put_* call writes them)."""
        if self.count + phases > self.max_phases:
            raise KernelError(f"a decode program of more than {self.max_phases} phases")

    def add(self, code: int, *tensors, activation_bytes: int = 0) -> None:
        """`code`: what a pae_program_put_* call returned (the bytes of LDS a quad needs, or an error);
        `activation_bytes`: the LDS a product's activations take (pae_program_activation_bytes)."""
        if code < 0:
            _check(code)
        self.room(1)
        self.count += 1
        self.quad_lds = max(self.quad_lds, code)
        self.activation_lds = max(self.activation_lds, activation_bytes)
        self.keep.append(tensors)  # what the phase reads and writes stays alive until the program has run

    def launch(self) -> None:
        if self.count == 0:
            return
        global _RECORDING
        assert _RECORDING is None, "a program is launched after its recording has ended"
        copy_int32_from_pinned(self.on_device, self.host, self.count * self.phase_bytes // 4)
        _check(library().pae_program_run(self.on_device.data_ptr(), self.count, self.barrier.data_ptr(),
                                         self.error.data_ptr(), self.groups, self.quad_lds, self.activation_lds,
                                         PROGRAM_SPIN_LIMIT, _ptr(self.trace), _stream()))
        if not torch.cuda.is_current_stream_capturing():
            self._read = self._read or torch.cuda.Event()
            self._read.record()

    def trace_phases(self) -> torch.Tensor:
        """From now on every launch leaves, per phase and workgroup, eight numbers: clock readings (100 MHz)
        [0] when it began the phase's work, [1] when it ended it (the difference to the next phase's
        beginning is its wait at the barrier), [2..5] marks of the phase's own (see pae_program_run; zero
        where a phase leaves none), and [7] the die that the workgroup ran on."""
        self.trace = torch.zeros((self.max_phases, self.groups, 8), dtype=torch.int64, device=self.device)
        return self.trace

    def check(self) -> None:
        """Raise if a launch of this program gave up at a barrier (call after the device has been waited for)."""
        code = int(self.error[0])
        if code:
            self.error[0] = 0
            self.barrier.zero_()
            skinny_tickets(self.device).zero_()
            raise KernelError(f"the decode program's workgroups did not all arrive at the barrier after phase {code - 1}: "
                              "the program was abandoned and its results are invalid")


class recording:
    """`with recording(program):` the product and decode-attention wrappers append phases to `program`."""

    def __init__(self, program: DecodeProgram) -> None:
        self.program = program

    def __enter__(self):
        global _RECORDING
        if _RECORDING is not None:
            raise KernelError("a decode program is already recording")
        self.program.begin()
        _RECORDING = self.program
        return self.program

    def __exit__(self, *exc):
        global _RECORDING
        _RECORDING = None
        return False


SKINNY_MAX_ROWS = 64
# Up to this many rows a norm may be folded into the products around it (see parts.OwedRows): as many as
# the few-rows products take (PAE_FOLD_MAX_ROWS: fewer, for a measurement).  Above 16 rows only while
# rows x width stays within FOLD_MAX_ELEMENTS.  Measured with the step itself: folding gains 2 to 6 % at 24
# to 64 rows of the 0.5B, 1.5B and 3B shapes (widths 896 to 2,048), 1.3 / 0.6 % at 24 / 32 rows of the 7B
# shape (3,584) and 2.6 % at 24 rows of the 14B shape (5,120), is even at 40 rows of the 7B shape and loses
# 1.7 / 1.2 % at its 48 / 64 rows, where the norm kernel is cheaper than the products' epilogues that stand
# in for it.
FOLD_MAX_ROWS = int(os.environ.get("PAE_FOLD_MAX_ROWS", "64"))
FOLD_MAX_ELEMENTS = 64 * 2048


def folds(rows: int, width: int) -> bool:
    """Whether a norm of `width` columns is folded into the products around it in a step of `rows` rows."""
    if not 0 < rows <= FOLD_MAX_ROWS:
        return False
    return rows <= SAME_ORDER_MAX_ROWS or rows * width <= FOLD_MAX_ELEMENTS


SAME_ORDER_MAX_ROWS = 16  # up to this many rows a product's k ranges depend on its sizes alone
EPI_BF16, EPI_F32, EPI_SWIGLU, EPI_RESIDUAL = 0, 1, 2, 4


def stat_tiles(width: int) -> int:
    """Shares a row's sum of squares is kept in: one per 16 columns."""
    return -(-width // 16)


def _row_scale(row_scale, M: int, K: int):
    """(pointer, tiles, eps) of the shares of the rows' sums of squares, for a product whose rows
    are still to be divided by their root mean square; (None, 0, 0) for plain rows."""
    if row_scale is None:
        return None, 0, 0.0
    stats, eps = row_scale
    assert stats.is_cuda and stats.dtype == torch.float32 and stats.is_contiguous()
    assert stats.dim() == 2 and stats.shape[0] >= M and stats.shape[1] == stat_tiles(K)
    return stats.data_ptr(), stats.shape[1], float(eps)


def embedding_rows(residual: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float,
                   next_rows: torch.Tensor, next_w: torch.Tensor, next_stats: torch.Tensor) -> None:
    """`embedding` for a step whose first norm is folded into the products: beside residual[t] =
    scale * table[ids[t]], next_rows[t] = bfloat16(residual[t] * next_w) and next_stats[t][j] = the sum
    of squares of residual[t] over columns 16 j .. 16 j + 15."""
    _not_while_recording("embedding_rows")
    _gpu(residual, table, ids, next_rows, next_w, next_stats)
    T, H = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous() and table.is_contiguous()
    assert ids.dtype == torch.int32 and ids.numel() == T and table.shape[1] == H
    assert next_rows.dtype == torch.bfloat16 and next_rows.shape == (T, H) and next_rows.is_contiguous()
    assert next_stats.dtype == torch.float32 and next_stats.shape == (T, stat_tiles(H)) and next_stats.is_contiguous()
    assert next_w.numel() == H
    wp, wf = _param(next_w)
    _check(library().pae_embedding_rows(code_of(table.dtype), residual.data_ptr(), table.data_ptr(), ids.data_ptr(),
                                        T, H, table.shape[0], float(scale), next_rows.data_ptr(), wp, wf,
                                        next_stats.data_ptr(), _stream()))


def scaled_rows(rows: torch.Tensor, stats: torch.Tensor, eps: float) -> torch.Tensor:
    """rows[m] * rsqrt(sum(stats[m]) / width + eps) as bfloat16: rows whose scale was owed, paid."""
    _not_while_recording("scaled_rows")
    _gpu(rows, stats)
    M, H = rows.shape
    assert rows.dtype == torch.bfloat16 and rows.is_contiguous()
    assert stats.dtype == torch.float32 and stats.shape == (M, stat_tiles(H)) and stats.is_contiguous()
    out = torch.empty_like(rows)
    _check(library().pae_scaled_rows(out.data_ptr(), rows.data_ptr(), stats.data_ptr(), stats.shape[1], float(eps),
                                     M, H, _stream()))
    return out


def skinny_supported(a: torch.Tensor, w: torch.Tensor) -> bool:
    """The weight-streaming product takes bfloat16, at most 64 rows and rows of 16-byte multiples."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[0] <= SKINNY_MAX_ROWS
            and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0 and a.stride(1) == 1 and a.data_ptr() % 16 == 0)


def skinny_splits(N: int, K: int, M: int = 1) -> int:
    """k ranges for a product whose consumer adds float32 partials: enough workgroups to fill the
    chip (a workgroup takes 16 weight rows, or 32 and more with more than 8 rows of activations)."""
    rows = 32 if M > 8 else 16
    tiles = -(-N // rows)
    # (ranges of at least 1,024 of k: the 0.5B sizes at 8 rows, O 5.3 us in three ranges and 3.9 in one, down
    # 8.0 us in eight and 7.4 in four)
    wanted = max(1, min(512 // tiles, K // 1024, 8))
    if M <= 8 and tiles >= 200 and tiles * wanted < 640 and K >= 4096:
        # one or two workgroups per compute unit, each with a long way to go (14B down at 8 rows:
        # 320 workgroups over 13,824 of k take 48 us with the norm, three ranges 35 us)
        wanted = min(8, -(-960 // tiles))
    if M > 8:
        # every range costs its partial sums a trip to memory and back in the norm that adds them, so a
        # workgroup wants about 128 KB of weights before another range pays (with the norm, at 64 rows:
        # 1.5B O one range 9.8 us, six 11.5; 1.5B down four 21.0, eight 22.9; 7B O two 18.2, four 19.8)
        wanted = max(1, min(8, round(rows * K * 2 / 131072)))
        # enough ranges of at least 1024 for the many-weight-rows kernel (128 rows a workgroup) to fill
        # the chip twice, where that many exist (72B down at 64 rows: 2 ranges 177 us, 8 ranges 115 us)
        groups = -(-N // 128)
        many = min(12, -(-512 // groups))
        while many > 1 and K // many < 1024:
            many -= 1
        if groups * many >= 256:
            wanted = max(wanted, many)
        # or fewer, longer ranges for that kernel's 64-row workgroups, where those fill the chip and the
        # 128-row ones do not (7B down at 48 rows: 12 ranges 47 us, 8 ranges of 64-row workgroups 42 us)
        # (ranges down to 768 of k: 14B/32B O, 5,120 x 5,120, at 24 / 64 rows from HBM with the norm: two ranges
        # 28.2 / 38.0 us, six 22.7 / 27.6)
        fewer = -(-448 // -(-N // 64))
        if fewer <= 8 and K // fewer >= 768 and groups * fewer < 256:
            wanted = fewer
        # or, with few weight rows, as many ranges as make one round of 32-row workgroups over the chip (3B
        # down, 64 x 4: 19.9 / 23.7 us with the norm against 23.1 / 29.0 with five ranges; 1.5B down, 48 x 5)
        one_round = _compute_units() // -(-N // 32)
        if M > SAME_ORDER_MAX_ROWS and 4 <= one_round <= 8 and K // one_round >= 1024:
            wanted = one_round
    k_per = -(-(-(-K // wanted)) // 128) * 128
    return -(-K // k_per)


_UNITS = 0


def _compute_units() -> int:
    global _UNITS
    if not _UNITS:
        _UNITS = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count if torch.cuda.is_available() else 256
    return _UNITS


def residual_splits(N: int, K: int, M: int = 1) -> int:
    """k ranges for a product that adds itself into the residual (EPI_RESIDUAL).  Up to 16 rows from
    the product's sizes alone: a row's sums are the same bits whatever it is batched with, launched by
    itself or as a phase of a decode program.  Four ranges run side by side in one workgroup of sixteen
    wavefronts, with no tickets and no trip to memory for partial sums, and are ahead wherever the 16-row
    workgroups fill the chip or have little to read (1.5B O at 8 rows 7.2 -> 5.9 us, 7B down 38.3 -> 36.1
    us, 72B down 111 -> 107.5 us); a few workgroups with much to read each want ticketed ranges (1.5B
    down: 96 workgroups of 287 KB, 17.4 us in one workgroup each, 12.5 in five ranges)."""
    if M > SAME_ORDER_MAX_ROWS:
        # Where norms are folded beyond that many rows (all from HBM, at 24 and 64 rows):
        groups32 = -(-N // 32)
        if groups32 <= 96 and K <= 6144:
            # few and short weight rows: one range, no tickets, the rows of A shared out over the workgroups
            # (0.5B down: 10.7 / 11.2 us against 15.5 / 19.6 in two ticketed ranges and 11.0 / 12.6 in seven)
            return 1
        # else the ranges of the partial-sum rule, which suit the residual epilogue as well (1.5B down, 48 x 5
        # workgroups: 15.6 / 17.9 us against 16.8 / 19.9 with four ranges; 3B down, 64 x 4: 18.5 / 22.9 against
        # 21.8 / 28.4 with five; 7B down: eight, 35 / 47 us; 14B: six, 33 / 44; 14B O: six, 19 / 27 against 27 / 37
        # with two)
        return skinny_splits(N, K, M)
    tiles = -(-N // 16)
    # one such workgroup fills a compute unit, so the tiles should fill the chip's units a whole number of
    # times, or nearly (14B/32B down: 320 tiles are a full round and a quarter of one; 32B at 8 rows 86.7 us
    # side by side, ticketed ranges are ahead)
    units = _compute_units()
    rounds_full = tiles <= units or tiles % units == 0 or tiles % units >= 3 * units // 4
    if K >= 1024 and (tiles >= 192 or 32 * K <= 65536) and rounds_full:
        return -(-K // (-(-(-(-K // 4)) // 128) * 128))  # four, as the rounding to 128 leaves them
    splits = skinny_splits(N, K, 1)
    if splits == 4 and K >= 1024 and (tiles >= 192 or 32 * K <= 65536):
        # four would be taken side by side (the same sums, slower here)
        return 5 if K // 5 >= 256 else 3
    return splits  # (four ticketed ranges where the launcher keeps them apart: 3B down at 8 rows 14.7 us, five 16.5)


def gemm_skinny(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                epilogue: int = EPI_BF16, splits: int = 1, row_scale=None, following=None) -> None:
    """out = a @ w^T for at most 64 rows of `a`, reading `w` once.

    EPI_BF16: out [M, N] bfloat16 (+bias).  EPI_F32: out [M, N] float32, or [splits, M, N]
    partial sums over k ranges.  EPI_SWIGLU: w holds blocks of 8 gate rows followed by their 8
    up rows; out [M, N / 2] = silu(gate) * up.  With several k ranges the other epilogues'
    partial sums are added up inside the kernel (see `skinny_tickets`).

    `row_scale = (stats, eps)`: the rows of `a` are bfloat16(x * w_norm) of rows x that are still
    to be divided by their root mean square; `stats[m]` holds shares that add up to sum(x[m]^2),
    and row m's sums are multiplied by rsqrt(that / K + eps) before the epilogue.
    EPI_RESIDUAL: `out` is the float32 residual [M, N], to which the product is added in place;
    `following = (next_rows, next_w, next_stats)` receives bfloat16(out * next_w) [M, N] and the
    shares [M, stat_tiles(N)] of the new rows' sums of squares, for the product after the next norm."""
    _gpu(out, a, w, bias)
    M, K_ = a.shape
    N = w.shape[0]
    assert skinny_supported(a, w) and w.shape == (N, K_) and w.is_contiguous() and out.is_contiguous()
    nr = nw = ns = None
    nwf, ld_next = 0, 0
    if epilogue == EPI_SWIGLU:
        assert out.shape == (M, N // 2) and out.dtype == torch.bfloat16 and bias is None
    elif epilogue == EPI_F32:
        assert out.dtype == torch.float32
        assert tuple(out.shape) == ((M, N) if splits == 1 and out.dim() == 2 else (splits, M, N))
    elif epilogue == EPI_RESIDUAL:
        assert out.shape == (M, N) and out.dtype == torch.float32 and bias is None and following is not None
        next_rows, next_w, next_stats = following
        _gpu(next_rows, next_w, next_stats)
        assert next_rows.dtype == torch.bfloat16 and next_rows.shape == (M, N) and next_rows.stride(1) == 1
        assert next_stats.dtype == torch.float32 and next_stats.shape == (M, stat_tiles(N)) and next_stats.is_contiguous()
        assert next_w.numel() == N
        nr, ns, ld_next = next_rows.data_ptr(), next_stats.data_ptr(), next_rows.stride(0)
        nw, nwf = _param(next_w)
    else:
        assert out.shape == (M, N) and out.dtype == torch.bfloat16
    bp, bf = _param(bias)
    sp, st, se = _row_scale(row_scale, M, K_)
    parts, counters = _ticket_scratch(a.device, M, N, splits if epilogue != EPI_F32 else 1)
    if _RECORDING is not None:
        _RECORDING.add(library().pae_program_put_product(
            _RECORDING.host_ptr, _RECORDING.count, epilogue, out.data_ptr(), out.stride(-2), a.data_ptr(), a.stride(0),
            w.data_ptr(), bp, bf, M, N, K_, splits, _ptr(parts), _ptr(counters), sp, st, se, nr, ld_next, nw, nwf, ns,
            None), out, a, w, bias, parts, row_scale, following,
            activation_bytes=library().pae_program_activation_bytes(M, K_, splits))
        return
    checking = (parts is not None and CHECK_TICKET_SUMS and not torch.cuda.is_current_stream_capturing())
    before = out.clone() if checking and epilogue == EPI_RESIDUAL else None
    _launch_ticketed(counters, lambda: library().pae_gemm_skinny(
        epilogue, out.data_ptr(), out.stride(-2), a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, N, K_, splits,
        M * N, _ptr(parts), _ptr(counters), sp, st, se, nr, ld_next, nw, nwf, ns, _stream()))
    if checking:
        _check_ticket_sums(out, before, a, w, bias, epilogue, splits, row_scale, following)


def gemm_skinny_act(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, kind: str, splits: int = 1,
                    bias: Optional[torch.Tensor] = None) -> None:
    """out [M, N] bfloat16 = act(a @ w^T + bias) for at most 64 rows of `a`: the weight-streaming product
    with the activation `kind` (see ACTIVATIONS) on its finished float32 sums, rounded once."""
    _not_while_recording("gemm_skinny_act")
    _gpu(out, a, w, bias)
    M, K_ = a.shape
    N = w.shape[0]
    assert skinny_supported(a, w) and w.shape == (N, K_) and w.is_contiguous() and out.is_contiguous()
    assert out.shape == (M, N) and out.dtype == torch.bfloat16 and kind in ACTIVATIONS
    bp, bf = _param(bias)
    parts, counters = _ticket_scratch(a.device, M, N, splits)
    _launch_ticketed(counters, lambda: library().pae_gemm_skinny_act(
        out.data_ptr(), out.stride(0), a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, N, K_, splits, _ptr(parts),
        _ptr(counters), ACTIVATIONS[kind], _stream()))


def gemm_skinny_gated(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, kind: str, splits: int = 1) -> None:
    """out [M, N / 2] bfloat16 = act(gate) * up for at most 64 rows of `a`, where w [N, K] holds blocks of 8
    gate rows followed by their 8 up rows (the layout of EPI_SWIGLU) and `kind` names the gate's activation."""
    _not_while_recording("gemm_skinny_gated")
    _gpu(out, a, w)
    M, K_ = a.shape
    N = w.shape[0]
    assert skinny_supported(a, w) and w.shape == (N, K_) and w.is_contiguous() and out.is_contiguous()
    assert N % 16 == 0 and out.shape == (M, N // 2) and out.dtype == torch.bfloat16 and kind in ACTIVATIONS
    parts, counters = _ticket_scratch(a.device, M, N, splits)
    _launch_ticketed(counters, lambda: library().pae_gemm_skinny_gated(
        out.data_ptr(), out.stride(0), a.data_ptr(), a.stride(0), w.data_ptr(), M, N, K_, splits, _ptr(parts),
        _ptr(counters), ACTIVATIONS[kind], _stream()))


# PAE_CHECK_TICKETS=sums: every product whose k ranges are added up inside the kernel is computed a
# second time in one k range (no tickets, no partial sums in memory) and the two results are compared.
# A partial sum read stale (from an earlier launch, or before it had arrived) is a whole k range's worth
# of error and shows far above the difference that the other order of adding leaves.
CHECK_TICKET_SUMS = os.environ.get("PAE_CHECK_TICKETS", "") == "sums"


def _check_ticket_sums(out, before, a, w, bias, epilogue, splits, row_scale, following) -> None:
    again = before if before is not None else torch.empty_like(out)
    follow = None
    if following is not None:
        follow = (torch.empty_like(following[0]), following[1], torch.empty_like(following[2]))
    pairs = [(out, again)] + ([(following[0], follow[0])] if follow is not None else [])
    gemm_skinny(again, a, w, bias, epilogue, 1, row_scale, follow)
    for got, want in pairs:
        got, want = got.float(), want.float()
        bound = 2.0 ** -6 * float(want.abs().max()) + 1e-30
        worst = float((got - want).abs().max())
        if not worst <= bound:
            raise KernelError(f"a product of {tuple(a.shape)} by {tuple(w.shape)} added up over {splits} k ranges inside "
                              f"the kernel differs from the same product in one range by {worst:.3e} (bound {bound:.3e}): "
                              "a partial sum was read before it had arrived, or left over from another launch")


TICKET_ARCHS = ("gfx950",)  # chips on which the fence-free ticket scheme has been validated
_TICKETS: dict = {}        # device index -> counters
_TICKET_STREAM: dict = {}  # device index -> the stream whose launches use them


def skinny_tickets(device) -> torch.Tensor:
    """The zeroed counters of products whose k ranges are added up inside the kernel.  Every launch
    leaves them zero, and launches share them, so they must run one after the other: the counters
    belong to the stream that is current when they are made (a model asks when it is bound, before
    any step is recorded as a graph), and `_ticket_scratch` refuses launches from another stream.
    Recording a graph on torch's capture stream is not a launch; its replays are, on the stream
    they are replayed on."""
    index = torch.device(device).index or 0
    if index not in _TICKETS:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("the ticket counters must exist before a graph is recorded")
        if device_arch() not in TICKET_ARCHS:
            # the scheme leans on how this chip's device-scope stores and loads reach the memory side
            # (see SkinnyTickets in csrc/gemm_skinny.hip); it has been validated on these chips only
            raise KernelError(f"k ranges added up inside a kernel are validated on {', '.join(TICKET_ARCHS)} only, "
                              f"not on {device_arch()}")
        _TICKETS[index] = torch.zeros(1 << 16, dtype=torch.int32, device=device)
        _TICKET_STREAM[index] = torch.cuda.current_stream(device).cuda_stream
    return _TICKETS[index]


def check_tickets_zero(device) -> None:
    """Raise unless every ticket counter is zero (it waits for the device: a check for tests and
    for runs with PAE_CHECK_TICKETS set, after each step)."""
    index = torch.device(device).index or 0
    counters = _TICKETS.get(index)
    if counters is not None and bool(counters.any()):
        where = counters.nonzero().flatten()[:8].tolist()
        raise KernelError(f"ticket counters {where} are not zero between launches: a product with k ranges "
                          "was cut short, or launches from two streams overlapped")


def _ticket_scratch(device, M: int, N: int, splits: int):
    """(partial sums, counters) for a product whose k ranges are added up inside the kernel."""
    if splits <= 1:
        return None, None
    lib, counters = library(), skinny_tickets(device)
    index = torch.device(device).index or 0
    if (not torch.cuda.is_current_stream_capturing()
            and torch.cuda.current_stream(device).cuda_stream != _TICKET_STREAM[index]):
        raise KernelError("products with k ranges share their ticket counters and must all be launched on the "
                          "stream the counters were made on; this launch comes from another stream")
    if lib.pae_skinny_ticket_slots(M, N) > counters.numel():
        raise KernelError(f"{N} weight rows by {M} rows need more ticket counters than there are")
    return torch.empty(lib.pae_skinny_ticket_floats(M, N, splits), dtype=torch.float32, device=device), counters


def _launch_ticketed(counters, call) -> None:
    """Run a launch that uses the ticket counters; if it is refused or fails, the counters are put
    back to zero before the error goes up (a later product would otherwise add up the wrong ranges)."""
    try:
        _check(call())
    except KernelError:
        if counters is not None and not torch.cuda.is_current_stream_capturing():
            counters.zero_()
        raise


def whole_sum_splits(N: int, K: int, M: int) -> int:
    """k ranges for a product whose epilogue needs whole sums (gate, rotation, bias), which the
    kernel then adds up itself.  That costs a trip to memory, and pays with more than 8 rows of
    activations where workgroups are few (measured at the 1.5B to 72B layer sizes):
    * the many-weight-rows kernel with little more than one workgroup per compute unit (7B gate/up
      at 64 rows: 85 -> 72 us; with more weight rows, or somewhat fewer, one range is as fast or faster);
    * few weight rows (the QKV products): ranges of about 1,280 (7B at 64 rows 26 -> 22 us in three,
      14B 37 -> 31 us in four, 72B 87 -> 54 us in six);
    * not with very few weight rows, where the rows of activations are shared out instead."""
    tiles, groups = -(-N // 32), -(-N // 128)
    if M <= SAME_ORDER_MAX_ROWS:
        # from the sizes alone, so that a row's sums do not depend on the batch (as `residual_splits`): one
        # range at every size (QKV from HBM at 1 / 8 / 16 rows, one range against the best of two to six: 72B
        # 37.2 / 43.7 / 52.0 us against 36.4 / 42.8 / 59.6; 14B 18.7 / 23.3 / 29.4 against 20.7 / 24.1 / 30.3; 7B 13.1 /
        # 15.2 / 20.4 against 13.1 / 14.1 / 20.9; gate/up likewise at all seven widths)
        return 1
    waves = -(-(-(-N // 16)) // 256)  # wavefronts of 16 weight rows a workgroup for at most 256 workgroups
    if 5 <= waves <= 8 and -(-(-(-N // 16)) // waves) >= 216:
        # one workgroup per compute unit, nearly all units busy: one range (the launcher then takes the
        # kernel of `waves` wavefronts; 1.5B gate/up at 32 rows 19.1 -> 16.7 us, at 64 rows 23.4 -> 22.2)
        return 1
    if 128 <= groups < 256:
        # a couple of workgroups of 32 weight rows per compute unit: three ranges from 32
        # rows on (1.5B gate/up at 64 rows 27.2 -> 23.3 us, at 32 rows 20.2 -> 19.0 us; below, one range is ahead)
        return 3 if M >= 32 and K >= 1536 else 1
    if tiles <= 96 or groups >= 384:
        return 1
    if groups >= 256:
        wanted = -(-(768 if M > 48 else 512) // groups)
        if K // wanted < 512:
            return 1
    else:
        # (and no more than make about a thousand 32-row workgroups: 72B QKV at 32 / 64 rows, 320 tiles, six
        # ranges 44.6 / 56.8 us, three 40.3 / 52.9)
        wanted = min(8, max(1, (K + 640) // 1280), max(1, round(1000 / tiles)))
    k_per = -(-(-(-K // wanted)) // 128) * 128
    return -(-K // k_per)


def skinny_rope_supported(a: torch.Tensor, w: torch.Tensor, hd: int, rot: int) -> bool:
    """Whether `gemm_skinny_rope` takes this product: a skinny product whose head size and
    rotated width are multiples of 16."""
    return skinny_supported(a, w) and hd % 16 == 0 and rot % 16 == 0 and 0 <= rot <= hd


def gemm_skinny_rope(q_out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], nh: int,
                     nkv: int, hd: int, rot: int, cos_sin: Optional[torch.Tensor], positions: torch.Tensor,
                     tok_seq: Optional[torch.Tensor], block_tables: Optional[torch.Tensor], block_size: int,
                     k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                     splits: Optional[int] = None, row_scale=None) -> None:
    """Query/key/value projection of at most 64 rows with the rotation and the cache write in its
    epilogue: q_out[M, nh * hd] = rotated queries; rotated keys and raw values go to their slots
    (nkv == 0: `w` holds the query rows only and nothing is stored).  `cos_sin`: see `rope_table`."""
    _gpu(q_out, a, w, bias, cos_sin, positions, tok_seq, block_tables, k_cache, v_cache)
    M, K_ = a.shape
    assert skinny_rope_supported(a, w, hd, rot) and w.shape == ((nh + 2 * nkv) * hd, K_) and w.is_contiguous()
    assert q_out.shape == (M, nh * hd) and q_out.dtype == torch.bfloat16 and q_out.stride(1) == 1
    assert positions.dtype == torch.int32 and positions.numel() == M
    _check_cos_sin(cos_sin, rot, M)
    max_blocks = 0
    if nkv:
        assert k_cache.dtype == torch.bfloat16 == v_cache.dtype
        assert tok_seq.dtype == torch.int32 and tok_seq.numel() == M
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        _check_pools(k_cache, v_cache, nkv, block_size, hd)
        max_blocks = block_tables.shape[1]
    bp, bf = _param(bias)
    lib, N = library(), w.shape[0]
    splits = 1 if splits is None else splits
    parts, counters = _ticket_scratch(a.device, M, N, splits)
    sp, st, se = _row_scale(row_scale, M, K_)
    if _RECORDING is not None:
        _RECORDING.add(lib.pae_program_put_product_rope(
            _RECORDING.host_ptr, _RECORDING.count, q_out.data_ptr(), q_out.stride(0), a.data_ptr(), a.stride(0),
            w.data_ptr(), bp, bf, M, K_, nh, nkv, hd, rot, _ptr(cos_sin) if rot else None, positions.data_ptr(),
            _ptr(tok_seq), _ptr(block_tables), max_blocks, block_size, _ptr(k_cache), _ptr(v_cache), splits, _ptr(parts),
            _ptr(counters), sp, st, se), q_out, a, w, bias, cos_sin, parts, row_scale,
            activation_bytes=lib.pae_program_activation_bytes(M, K_, splits))
        return
    _launch_ticketed(counters, lambda: lib.pae_gemm_skinny_rope(
        q_out.data_ptr(), q_out.stride(0), a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, K_, nh, nkv, hd, rot,
        _ptr(cos_sin) if rot else None, positions.data_ptr(), _ptr(tok_seq), _ptr(block_tables), max_blocks,
        block_size, _ptr(k_cache), _ptr(v_cache), splits, _ptr(parts), _ptr(counters), sp, st, se, _stream()))


def gemm_plain(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias), float32 accumulation in k order."""
    _not_while_recording("gemm_plain")
    _gpu(out, a, w, bias)
    M, K = a.shape
    N = w.shape[0]
    assert w.shape == (N, K) and w.is_contiguous() and w.dtype == a.dtype
    assert out.shape == (M, N) and a.stride(1) == 1 and out.stride(1) == 1
    if bias is not None:
        assert bias.numel() == N
    bp, bf = _param(bias)
    _check(library().pae_gemm_plain(code_of(a.dtype), code_of(out.dtype), out.data_ptr(), out.stride(0),
                                    a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, N, K, _stream()))


def gemm_plain_heads(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor) -> None:
    """One product per head: out[:, h, :] = a[:, h, :] @ w[h]^T, float32 accumulation in k order.
    `a` [M, B, K] and `out` [M, B, N] are views whose last dimension is contiguous (heads of wider
    rows, say); `w` [B, N, K] is contiguous."""
    _not_while_recording("gemm_plain_heads")
    _gpu(out, a, w)
    M, B, K = a.shape
    N = w.shape[1]
    assert w.shape == (B, N, K) and w.is_contiguous() and w.dtype == a.dtype
    assert out.shape == (M, B, N) and a.stride(2) == 1 and out.stride(2) == 1
    _check(library().pae_gemm_plain_batched(code_of(a.dtype), code_of(out.dtype), out.data_ptr(), out.stride(0),
                                            out.stride(1), a.data_ptr(), a.stride(0), a.stride(1), w.data_ptr(),
                                            w.stride(0), None, 0, M, N, K, B, _stream()))


HEADS_FEW_MAX_ROWS = 16


def heads_product(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor) -> None:
    """out[:, h, :] = a[:, h, :] @ w[h]^T for every head h (shapes as for `gemm_plain_heads`).  bfloat16 with
    more rows than the few-row kernels take goes to the platform's batched matrix product, as the plain
    products of that many rows do; bfloat16 with up to 16 rows to a kernel that streams the weights once;
    everything else to the plain product's batched entry."""
    if a.dtype == torch.bfloat16 and 0 < a.shape[0] <= HEADS_FEW_MAX_ROWS:
        # a few rows: one wavefront per (head, output feature), the weights read once (every wavefront reads all rows
        # of its head: at 64 rows that costs more than the plain kernel's tiles, measured)
        _not_while_recording("heads_product")
        _gpu(out, a, w)
        M, B, K_ = a.shape
        N = w.shape[1]
        assert w.shape == (B, N, K_) and w.is_contiguous() and w.dtype == a.dtype == out.dtype
        assert out.shape == (M, B, N) and a.stride(2) == 1 and out.stride(2) == 1
        _check(library().pae_heads_product_few(out.data_ptr(), out.stride(0), out.stride(1), a.data_ptr(), a.stride(0),
                                               a.stride(1), w.data_ptr(), M, N, K_, B, _stream()))
        return
    if a.dtype == torch.bfloat16 and a.shape[0] > SKINNY_MAX_ROWS and _RECORDING is None:
        # [B, M, K] x [B, K, N] on strided views: no copy of the operands; the result is copied into the view
        out.copy_(torch.bmm(a.transpose(0, 1), w.transpose(1, 2)).transpose(0, 1))
        return
    gemm_plain_heads(out, a, w)


def paged_attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            positions: torch.Tensor, tok_seq: torch.Tensor, block_tables: torch.Tensor,
                            nh: int, nkv: int, hd: int, scale: float, window: int) -> None:
    """out[t, h*hd:(h+1)*hd] = attention of query head h of token t over the cached
    keys start..positions[t] of sequence tok_seq[t]."""
    _not_while_recording("paged_attention_generic")
    _gpu(out, q, k_cache, v_cache, positions, tok_seq, block_tables)
    T = q.shape[0]
    bs = k_cache.shape[2]
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd and q.dtype == k_cache.dtype == out.dtype
    assert out.shape[0] == T and out.stride(1) == 1 and out.shape[1] >= nh * hd
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    _check(library().pae_paged_attention_generic(
        code_of(q.dtype), out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(),
        v_cache.data_ptr(), positions.data_ptr(), tok_seq.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], bs, T, nh, nkv, hd, float(scale), int(window), _stream()))


def _check_pools_wide(k_cache, v_cache, nkv: int, bs: int, hd: int, vd: int) -> None:
    """Keys [block][kv head][bs][hd]; values of width vd transposed within the page, [block][kv head][vd][bs]."""
    assert tuple(k_cache.shape[1:]) == (nkv, bs, hd) and k_cache.is_contiguous()
    assert tuple(v_cache.shape) == (k_cache.shape[0], nkv, vd, bs) and v_cache.is_contiguous()
    assert k_cache.dtype == v_cache.dtype


def paged_attention_capped(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           positions: torch.Tensor, tok_seq: torch.Tensor, block_tables: torch.Tensor,
                           nh: int, nkv: int, hd: int, vd: int, scale: float, window: int, softcap: float = 0.0,
                           sinks: Optional[torch.Tensor] = None) -> None:
    """`paged_attention_generic` with values of width `vd` (out[t, h*vd:(h+1)*vd]), scores capped by
    softcap * tanh(s / softcap) (0: no cap) and one sink per query head in the softmax's denominator
    (`sinks` float32 [nh], None: no sinks)."""
    _not_while_recording("paged_attention_capped")
    _gpu(out, q, k_cache, v_cache, positions, tok_seq, block_tables, sinks)
    T = q.shape[0]
    bs = k_cache.shape[2]
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd and q.dtype == k_cache.dtype == out.dtype
    assert out.shape[0] == T and out.stride(1) == 1 and out.shape[1] >= nh * vd
    _check_pools_wide(k_cache, v_cache, nkv, bs, hd, vd)
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == nh and sinks.is_contiguous()
    _check(library().pae_paged_attention_capped(
        code_of(q.dtype), out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(),
        v_cache.data_ptr(), positions.data_ptr(), tok_seq.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], bs, T, nh, nkv, hd, vd, float(scale), int(window), float(softcap), _ptr(sinks),
        _stream()))


def paged_attention_masked(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: Optional[torch.Tensor],
                           positions: torch.Tensor, tok_seq: torch.Tensor, block_tables: torch.Tensor,
                           nh: int, nkv: int, hd: int, vd: int, scale: float, window: int = 0, chunked: bool = False,
                           slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                           softcap: float = 0.0, sinks: Optional[torch.Tensor] = None) -> None:
    """`paged_attention_capped` with, each optional: the `window` read as a chunk length (`chunked`:
    position p sees keys from p - p % window on), a bias by distance (score -= slopes[h] * (p - key),
    float32 [nh]), and an output gate (out *= sigmoid(gate), `gate` a [T, >= nh * vd] view of rows).
    `v_cache` None: the values are the first `vd` features of the key rows, which are then one row
    per token, `k_cache` [block][bs][hd] (nkv must be 1)."""
    _not_while_recording("paged_attention_masked")
    _gpu(out, q, k_cache, v_cache, positions, tok_seq, block_tables, sinks, slopes, gate)
    T = q.shape[0]
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd and q.dtype == k_cache.dtype == out.dtype
    assert out.shape[0] == T and out.stride(1) == 1 and out.shape[1] >= nh * vd
    if v_cache is None:
        assert nkv == 1 and k_cache.dim() == 3 and k_cache.shape[2] == hd and k_cache.is_contiguous() and vd <= hd
        bs = k_cache.shape[1]
    else:
        bs = k_cache.shape[2]
        _check_pools_wide(k_cache, v_cache, nkv, bs, hd, vd)
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    for t in (sinks, slopes):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == nh and t.is_contiguous()
    gate_stride = 0
    if gate is not None:
        assert gate.dim() == 2 and gate.shape[0] == T and gate.stride(1) == 1 and gate.shape[1] >= nh * vd
        assert gate.dtype == q.dtype
        gate_stride = gate.stride(0)
    _check(library().pae_paged_attention_masked(
        code_of(q.dtype), out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(),
        _ptr(v_cache), positions.data_ptr(), tok_seq.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], bs, T, nh, nkv, hd, vd, float(scale), int(window), float(softcap), _ptr(sinks),
        1 if chunked else 0, _ptr(slopes), _ptr(gate), gate_stride, 1 if v_cache is None else 0, _stream()))


def conv_norm_store(proj: torch.Tensor, q_out: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor,
                    seq_runs: torch.Tensor, slots: torch.Tensor, conv_w: torch.Tensor, conv_tail: Optional[torch.Tensor],
                    taps: int, nh: int, nkv: int, hd: int, vd: int, norm_heads: bool, eps: float,
                    block_tables: Optional[torch.Tensor], block_size: int, k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor]) -> None:
    """Rows `proj` [T, >= C], C = nh hd + nkv (hd + vd), hold per token [q | k | v | anything else]:
    every one of the C channels passes a causal convolution of `taps` taps over the sequence's own
    tokens (`conv_w` float32 [C, taps]; inputs before the step from `conv_tail` float32
    [slots, taps - 1, C], which is moved on), then, with `norm_heads`, q and k heads are divided by
    their root mean square over hd.  Queries to `q_out` [T, nh * hd], keys and values to their cache
    slots (nkv = 0: queries only, no pools).  `seq_runs` int32 [S, 4] = (first row, rows, tokens
    before, 0) per sequence."""
    _not_while_recording("conv_norm_store")
    _gpu(proj, q_out, tok_seq, positions, seq_runs, slots, conv_w, conv_tail, block_tables, k_cache, v_cache)
    T, S = proj.shape[0], seq_runs.shape[0]
    C = nh * hd + nkv * (hd + vd)
    assert proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= C
    assert q_out.shape == (T, nh * hd) and q_out.stride(1) == 1 and q_out.dtype == proj.dtype
    for t, n in ((tok_seq, T), (positions, T), (slots, S)):
        assert t.dtype == torch.int32 and t.numel() >= n and t.is_contiguous()
    assert seq_runs.dtype == torch.int32 and seq_runs.shape == (S, 4) and seq_runs.is_contiguous()
    assert seq_runs.data_ptr() % 16 == 0
    assert conv_w.dtype == torch.float32 and conv_w.shape == (C, taps) and conv_w.is_contiguous()
    tail_stride = 0
    if taps > 1:
        assert conv_tail is not None and conv_tail.dtype == torch.float32
        assert tuple(conv_tail.shape[1:]) == (taps - 1, C) and conv_tail[0].is_contiguous()
        tail_stride = conv_tail.stride(0)
    max_blocks = 0
    if nkv:
        assert k_cache.dtype == proj.dtype == v_cache.dtype
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        assert block_tables.shape[0] >= S
        _check_pools_wide(k_cache, v_cache, nkv, block_size, hd, vd)
        max_blocks = block_tables.shape[1]
    _check(library().pae_conv_norm_store(
        code_of(proj.dtype), proj.data_ptr(), proj.stride(0), q_out.data_ptr(), q_out.stride(0), T, S,
        tok_seq.data_ptr(), positions.data_ptr(), seq_runs.data_ptr(), slots.data_ptr(), conv_w.data_ptr(),
        _ptr(conv_tail) if taps > 1 else None, tail_stride, taps, nh, nkv, hd, vd, 1 if norm_heads else 0, float(eps),
        _ptr(block_tables) if nkv else None, max_blocks, block_size, _ptr(k_cache) if nkv else None,
        _ptr(v_cache) if nkv else None, _stream()))


def latent_prepare(proj: torch.Tensor, q_full: torch.Tensor, nh: int, nope: int, rd: int, rot: int, interleaved: bool,
                   rank: int, norm_w: torch.Tensor, eps: float, cos_sin: Optional[torch.Tensor], positions: torch.Tensor,
                   tok_seq: torch.Tensor, block_tables: torch.Tensor, latent: torch.Tensor,
                   latent_t: Optional[torch.Tensor] = None) -> None:
    """Rows `proj` [T, nh (nope + rd) + rank + rd] = [query heads | down projection]: the first `rank`
    features of the down projection are RMS-normed with `norm_w` and, with the last rd (their first
    `rot` rotated by `cos_sin`), written to the token's row of `latent` [block][bs][rank + rd]; the
    query heads' last rd features are rotated likewise into q_full[t, h, rank:] (`q_full`
    [T, nh * (rank + rd)], whose first `rank` features per head the caller fills).  With `latent_t`
    [block][rank][bs] the normed latents are also written transposed within the page."""
    _not_while_recording("latent_prepare")
    _gpu(proj, q_full, norm_w, cos_sin, positions, tok_seq, block_tables, latent, latent_t)
    if latent_t is not None:
        assert tuple(latent_t.shape) == (latent.shape[0], rank, latent.shape[1]) and latent_t.is_contiguous()
        assert latent_t.dtype == latent.dtype
    T = proj.shape[0]
    assert proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= nh * (nope + rd) + rank + rd
    assert q_full.shape == (T, nh * (rank + rd)) and q_full.stride(1) == 1 and q_full.dtype == proj.dtype
    assert latent.dim() == 3 and latent.shape[2] == rank + rd and latent.is_contiguous() and latent.dtype == proj.dtype
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    assert norm_w.numel() == rank and norm_w.is_contiguous()
    _check_cos_sin(cos_sin, rot, T)
    wp, wf = _param(norm_w)
    _check(library().pae_latent_prepare(
        code_of(proj.dtype), proj.data_ptr(), proj.stride(0), q_full.data_ptr(), q_full.stride(0), T, nh, nope, rd, rot,
        1 if interleaved else 0, rank, wp, wf, float(eps), _ptr(cos_sin) if rot else None, positions.data_ptr(),
        tok_seq.data_ptr(), block_tables.data_ptr(), block_tables.shape[1], latent.shape[1], latent.data_ptr(),
        _ptr(latent_t), _stream()))


def latent_attn_supported(dtype: torch.dtype, row_width: int, rank: int, block_size: int = 16) -> bool:
    """Shapes the matrix-core latent attention takes; others go through the kernel for any shape."""
    return dtype == torch.bfloat16 and bool(library().pae_latent_attn_supported(row_width, rank, block_size))


def latent_attn_tokens(num_heads: int, column_tiles: int) -> int:
    """Tokens one workgroup of the matrix-core latent attention takes with that many tiles of 16 columns."""
    return library().pae_latent_attn_columns(num_heads, column_tiles)


def latent_attn(out: torch.Tensor, q_full: torch.Tensor, latent: torch.Tensor, latent_t: torch.Tensor, tiles: torch.Tensor,
                column_tiles: int, positions: torch.Tensor, block_tables: torch.Tensor, nh: int, rank: int, scale: float,
                window: int = 0, chunked: bool = False, sinks: Optional[torch.Tensor] = None) -> None:
    """Latent attention on the matrix cores.  `q_full` [T, nh * KD] holds per head the query folded into
    latent space and its rotated part; `latent` [block][bs][KD] and `latent_t` [block][rank][bs] are the
    cached rows and their transposed latents; tiles[i] = (table row, first flat token, tokens, 0) with at
    most `latent_attn_tokens(nh, column_tiles)` tokens; out[t, h * rank:(h + 1) * rank] receives the
    weighted sums of the latents.  `sinks` float32 [nh]: exp(sink) joins each head's denominator."""
    _not_while_recording("latent_attn")
    _gpu(out, q_full, latent, latent_t, tiles, positions, block_tables, sinks)
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == nh and sinks.is_contiguous()
    T = q_full.shape[0]
    kd, bs = latent.shape[2], latent.shape[1]
    assert q_full.dtype == torch.bfloat16 == out.dtype == latent.dtype == latent_t.dtype
    assert q_full.stride(1) == 1 and out.stride(1) == 1 and q_full.shape[1] >= nh * kd and out.shape[1] >= nh * rank
    assert out.shape[0] == T and latent.is_contiguous() and latent_t.is_contiguous()
    assert tuple(latent_t.shape) == (latent.shape[0], rank, bs)
    assert tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous()
    assert tiles.data_ptr() % 16 == 0
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    part_acc = part_ml = None
    splits = -(-block_tables.shape[1] * bs // library().pae_latent_attn_split())
    if column_tiles == 1 and splits > 1:
        # single tokens with tables beyond one split: the keys are shared out over workgroups and merged
        part_acc = torch.empty((tiles.shape[0] * splits * nh, rank), dtype=torch.float32, device=out.device)
        part_ml = torch.empty((tiles.shape[0] * splits * nh, 2), dtype=torch.float32, device=out.device)
    _check(library().pae_latent_attn_bf16(
        out.data_ptr(), out.stride(0), q_full.data_ptr(), q_full.stride(0), latent.data_ptr(), latent_t.data_ptr(),
        tiles.data_ptr(), tiles.shape[0], column_tiles, positions.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
        bs, nh, kd, rank, float(scale), int(window), 1 if chunked else 0, _ptr(part_acc), _ptr(part_ml), _ptr(sinks),
        _stream()))


def hyper_norm(streams: torch.Tensor, num_streams: int, y: Optional[torch.Tensor], layer_scale: Optional[torch.Tensor],
               mix: Optional[torch.Tensor], out_weights: Optional[torch.Tensor], in_weights: torch.Tensor,
               weight: torch.Tensor, eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
    """A stream kept as `num_streams` float32 copies per token (`streams` [T, S * H]).  With `y`, the
    pending branch output ([T, H] in out's dtype, or float32 partial sums [P, T, H]), all copies move
    on at once: x_t <- sum_s mix[s, t] x_s + out_weights[t] * (layer_scale * y).  Then
    out = rmsnorm(sum_s in_weights[s] x_s) * weight.  `mix` [S, S], `out_weights` and `in_weights` [S]
    are float32.  With `rows` (int32) only those rows are produced and nothing is written back."""
    _not_while_recording("hyper_norm")
    _gpu(streams, y, layer_scale, mix, out_weights, in_weights, weight, out, rows)
    S = num_streams
    T = streams.shape[0]
    H = out.shape[-1]
    n = out.shape[0]
    assert streams.dtype == torch.float32 and streams.is_contiguous() and tuple(streams.shape) == (T, S * H)
    assert out.is_contiguous() and weight.numel() == H
    assert in_weights.dtype == torch.float32 and in_weights.numel() == S and in_weights.is_contiguous()
    parts, part_stride = 0, 0
    if y is not None:
        assert y.is_contiguous()
        if y.dim() == 3:
            assert y.dtype == torch.float32 and tuple(y.shape[1:]) == (T, H)
            parts, part_stride = y.shape[0], T * H
        else:
            assert y.dtype == out.dtype and tuple(y.shape) == (T, H)
        assert mix.dtype == torch.float32 and tuple(mix.shape) == (S, S) and mix.is_contiguous()
        assert out_weights.dtype == torch.float32 and out_weights.numel() == S and out_weights.is_contiguous()
        if layer_scale is not None:
            assert layer_scale.numel() == H and layer_scale.is_contiguous()
    if rows is None:
        assert n == T
    else:
        assert rows.dtype == torch.int32 and rows.numel() == n
    lp, lf = _param(layer_scale if y is not None else None)
    wp, wf = _param(weight)
    _check(library().pae_hyper_norm(code_of(out.dtype), streams.data_ptr(), S, _ptr(y), parts, part_stride, lp, lf,
                                    _ptr(mix) if y is not None else None, _ptr(out_weights) if y is not None else None,
                                    in_weights.data_ptr(), wp, wf, float(eps), _ptr(rows), out.data_ptr(), n, H,
                                    0 if rows is not None else 1, _stream()))


def hyper_spread(streams: torch.Tensor, src: torch.Tensor, num_streams: int) -> None:
    """streams[t] = `num_streams` copies of src[t] (float32 [T, H] -> [T, S * H])."""
    _not_while_recording("hyper_spread")
    _gpu(streams, src)
    T, H = src.shape
    assert src.dtype == torch.float32 == streams.dtype and src.is_contiguous() and streams.is_contiguous()
    assert tuple(streams.shape) == (T, num_streams * H)
    _check(library().pae_hyper_spread(streams.data_ptr(), src.data_ptr(), T, num_streams, H, _stream()))


def hyper_collapse(streams: torch.Tensor, num_streams: int) -> torch.Tensor:
    """The sum of a token's copies: float32 [T, S * H] -> [T, H]."""
    _not_while_recording("hyper_collapse")
    _gpu(streams)
    T, H = streams.shape[0], streams.shape[1] // num_streams
    assert streams.dtype == torch.float32 and streams.is_contiguous() and streams.shape[1] == num_streams * H
    out = torch.empty((T, H), dtype=torch.float32, device=streams.device)
    _check(library().pae_hyper_collapse(out.data_ptr(), streams.data_ptr(), T, num_streams, H, _stream()))
    return out


def qk_norm_rotate_store(qkv: torch.Tensor, nh: int, nkv: int, hd: int, vd: int, q_weight: Optional[torch.Tensor],
                         k_weight: Optional[torch.Tensor], eps: float, rot: int, interleaved: bool,
                         cos_sin: Optional[torch.Tensor], magnitude: float, positions: torch.Tensor,
                         tok_seq: Optional[torch.Tensor], block_tables: Optional[torch.Tensor], block_size: int,
                         k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], per_head: bool = False) -> None:
    """Rows [q: nh x hd | k: nkv x hd | v: nkv x vd]: with weights, q and k are each divided by the root
    mean square of their whole projection and multiplied by the weight (`per_head`: every head by its own root
    mean square, and the weights are hd numbers that the heads share); the first `rot` features of
    every q and k head are rotated by `cos_sin` times `magnitude` (pairs (2i, 2i+1) if `interleaved`,
    else (i, i + rot/2)); queries are written back in place, keys and values to their cache slots
    (`k_cache` None: nkv must be 0 and nothing is stored)."""
    _not_while_recording("qk_norm_rotate_store")
    _gpu(qkv, q_weight, k_weight, cos_sin, positions, tok_seq, block_tables, k_cache, v_cache)
    T = qkv.shape[0]
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and positions.dtype == torch.int32 and positions.numel() == T
    write = k_cache is not None
    assert write or nkv == 0
    _check_cos_sin(cos_sin, rot, T)
    wf = 0
    if q_weight is not None:
        assert q_weight.numel() == (hd if per_head else nh * hd) and q_weight.is_contiguous()
        assert nkv == 0 or (k_weight is not None and k_weight.numel() == (hd if per_head else nkv * hd)
                            and k_weight.dtype == q_weight.dtype and k_weight.is_contiguous())
        wf = _param(q_weight)[1]
    max_blocks = 0
    if write:
        assert k_cache.dtype == qkv.dtype == v_cache.dtype
        assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        _check_pools_wide(k_cache, v_cache, nkv, block_size, hd, vd)
        max_blocks = block_tables.shape[1]
    _check(library().pae_qk_norm_rotate_store(
        code_of(qkv.dtype), qkv.data_ptr(), qkv.stride(0), T, nh, nkv, hd, vd, _ptr(q_weight), _ptr(k_weight), wf,
        float(eps), rot, 1 if interleaved else 0, _ptr(cos_sin) if rot else None, float(magnitude),
        positions.data_ptr(), _ptr(tok_seq), _ptr(block_tables), max_blocks, block_size, _ptr(k_cache), _ptr(v_cache),
        1 if write else 0, 1 if (per_head and q_weight is not None) else 0, _stream()))


def rows_from_residual(residual: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 stream [T, H] as rows of `dtype` for a matrix product (float32: the stream itself)."""
    _not_while_recording("rows_from_residual")
    _gpu(residual)
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    if dtype == torch.float32:
        return residual
    out = torch.empty(residual.shape, dtype=dtype, device=residual.device)
    _check(library().pae_rows_from_residual(code_of(dtype), out.data_ptr(), residual.data_ptr(), residual.numel(),
                                            _stream()))
    return out


def norm_scale_add(residual: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, scale: float,
                   next_rows: Optional[torch.Tensor] = None) -> None:
    """residual[t] += scale * y[t] / sqrt(mean(y[t]^2) + eps) * weight.  `y`: [T, H] in the activation
    type, or float32 partial sums [P, T, H] added in order.  `next_rows` [T, H] (the type of the
    activations) receives the new residual rounded to it."""
    _not_while_recording("norm_scale_add")
    _gpu(residual, y, weight, next_rows)
    T, H = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous() and y.is_contiguous()
    parts, stride = 0, 0
    if y.dim() == 3:
        assert y.dtype == torch.float32 and tuple(y.shape[1:]) == (T, H)
        parts, stride = y.shape[0], T * H
        dtype = next_rows.dtype if next_rows is not None else torch.bfloat16
    else:
        assert tuple(y.shape) == (T, H)
        dtype = y.dtype
    if next_rows is not None:
        assert tuple(next_rows.shape) == (T, H) and next_rows.is_contiguous() and next_rows.dtype == dtype
    assert weight.numel() == H
    wp, wf = _param(weight)
    _check(library().pae_norm_scale_add(code_of(dtype), residual.data_ptr(), y.data_ptr(), parts, stride, wp, wf,
                                        float(eps), float(scale), _ptr(next_rows), T, H, _stream()))


ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2}


def activation(x: torch.Tensor, kind: str) -> None:
    """x <- act(x) in place, computed in float32: "gelu" (by erf), "gelu_tanh", "silu"."""
    _not_while_recording("activation")
    _gpu(x)
    assert x.is_contiguous() and kind in ACTIVATIONS
    _check(library().pae_activation(code_of(x.dtype), x.data_ptr(), x.numel(), ACTIVATIONS[kind], _stream()))


def delta_rule_step(proj: torch.Tensor, out: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor,
                    seq_runs: torch.Tensor, slots: torch.Tensor, conv_w: torch.Tensor, conv_tail: torch.Tensor,
                    state: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, norm_w: torch.Tensor,
                    G: int, H: int, D: int, V: int, taps: int, unit_eps: float, norm_eps: float,
                    gate: Optional[torch.Tensor] = None, beta: Optional[torch.Tensor] = None,
                    decay_in: Optional[torch.Tensor] = None, channel_decay: bool = False,
                    gate_activation: str = "silu") -> None:
    """The gated delta rule over a step's rows.  `proj` [T, >= 2GD + HV] holds per token [q | k | v | ...];
    the gate's rows [T, HV], beta's [T, H] and the decay's input [T, H] come as views of rows in proj's type
    (`gate`, `beta`, `decay_in`), or, when none is given, from proj's tail [gate | b | a].  `seq_runs` int32
    [S, 4] = (first row, rows, tokens before, 0) per sequence; `slots` int32 [S]; `conv_w` float32
    [2GD + HV, taps]; `conv_tail` float32 [slots, taps - 1, 2GD + HV] and `state` float32 [slots, H, V, D] are
    the requests' state, read and moved on; `out` [T, H * V] receives the normed, gated read-out in proj's type.
    `channel_decay`: one decay per head and key channel (`decay_in` [T, H * D], `dt_bias` [H * D]) instead of
    one per head; `gate_activation`: "silu" or "sigmoid"."""
    _not_while_recording("delta_rule_step")
    _gpu(proj, out, tok_seq, positions, seq_runs, slots, conv_w, conv_tail, state, a_log, dt_bias, norm_w, gate, beta,
         decay_in)
    T, S = proj.shape[0], seq_runs.shape[0]
    C = 2 * G * D + H * V
    assert gate_activation in ("silu", "sigmoid")
    assert proj.dim() == 2 and proj.stride(1) == 1
    if gate is None and beta is None and decay_in is None:
        assert proj.shape[1] == C + H * V + 2 * H and not channel_decay
        gate, beta, decay_in = proj[:, C:C + H * V], proj[:, C + H * V:C + H * V + H], proj[:, C + H * V + H:]
    assert proj.shape[1] >= C
    for view, width in ((gate, H * V), (beta, H), (decay_in, H * D if channel_decay else H)):
        assert view is not None and view.dim() == 2 and view.shape == (T, width) and view.dtype == proj.dtype
        assert view.stride(1) == 1 or width == 1
    assert out.shape == (T, H * V) and out.is_contiguous() and out.dtype == proj.dtype
    for t, n in ((tok_seq, T), (positions, T), (slots, S)):
        assert t.dtype == torch.int32 and t.numel() >= n and t.is_contiguous()
    assert seq_runs.dtype == torch.int32 and seq_runs.shape == (S, 4) and seq_runs.is_contiguous()
    assert seq_runs.data_ptr() % 16 == 0
    assert conv_w.dtype == torch.float32 and conv_w.shape == (C, taps) and conv_w.is_contiguous()
    assert conv_tail.dtype == torch.float32 and tuple(conv_tail.shape[1:]) == (max(taps - 1, 0), C)
    assert conv_tail.stride(2) == 1 and (taps == 1 or conv_tail.stride(1) == C)
    assert state.dtype == torch.float32 and tuple(state.shape[1:]) == (H, V, D) and state[0].is_contiguous()
    assert state.shape[0] == conv_tail.shape[0]
    assert a_log.dtype == torch.float32 and a_log.numel() == H and a_log.is_contiguous()
    assert dt_bias.dtype == torch.float32 and dt_bias.numel() == (H * D if channel_decay else H) and dt_bias.is_contiguous()
    assert norm_w.numel() == V
    wp, wf = _param(norm_w)
    lib = library()
    work = torch.empty(lib.pae_delta_rule_work_floats(T, G, H, D, V, 1 if channel_decay else 0), dtype=torch.float32,
                       device=proj.device)
    _check(lib.pae_delta_rule_step(
        code_of(proj.dtype), proj.data_ptr(), proj.stride(0), T, S, tok_seq.data_ptr(), positions.data_ptr(),
        seq_runs.data_ptr(), slots.data_ptr(), conv_w.data_ptr(), conv_tail.data_ptr(), conv_tail.stride(0), taps, G, H,
        D, V, a_log.data_ptr(), dt_bias.data_ptr(), float(unit_eps), state.data_ptr(), state.stride(0), wp, wf,
        float(norm_eps), work.data_ptr(), out.data_ptr(), gate.data_ptr(), gate.stride(0),
        1 if gate_activation == "sigmoid" else 0, beta.data_ptr(), beta.stride(0), decay_in.data_ptr(), decay_in.stride(0),
        1 if channel_decay else 0, _stream()))


def matrix_memory_step(proj: torch.Tensor, gate: torch.Tensor, gate_logits: torch.Tensor, out: torch.Tensor,
                       seq_runs: torch.Tensor, slots: torch.Tensor, state: torch.Tensor, maximum: torch.Tensor,
                       norm_w: torch.Tensor, H: int, D: int, V: int, gate_cap: float, norm_eps: float,
                       floor_eps: float) -> None:
    """A matrix memory with exponential gates over a step's rows.  `proj` [T, >= 2HD + HV] holds per token
    [q | k | v]; `gate` [T, HV] (a view of rows in proj's type) is the output gate's input; `gate_logits` float32
    [T, 2H] the input and forget gates' sums with their biases.  `state` float32 [slots, H, V + 1, D] (the
    memory, and as its last column the sum of gated keys) and `maximum` float32 [slots, H] are the requests'
    state, read and moved on; `out` [T, H * V] receives o / (max(|n . q|, exp(-m)) + floor_eps), normed over V,
    times `norm_w` [H * V] and sigmoid(gate), in proj's type."""
    _not_while_recording("matrix_memory_step")
    _gpu(proj, gate, gate_logits, out, seq_runs, slots, state, maximum, norm_w)
    T, S = proj.shape[0], seq_runs.shape[0]
    assert proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= 2 * H * D + H * V
    assert gate.shape == (T, H * V) and gate.stride(1) == 1 and gate.dtype == proj.dtype
    assert gate_logits.dtype == torch.float32 and gate_logits.shape == (T, 2 * H) and gate_logits.is_contiguous()
    assert out.shape == (T, H * V) and out.is_contiguous() and out.dtype == proj.dtype
    assert slots.dtype == torch.int32 and slots.numel() >= S and slots.is_contiguous()
    assert seq_runs.dtype == torch.int32 and seq_runs.shape == (S, 4) and seq_runs.is_contiguous()
    assert seq_runs.data_ptr() % 16 == 0
    assert state.dtype == torch.float32 and tuple(state.shape[1:]) == (H, V + 1, D) and state[0].is_contiguous()
    assert maximum.dtype == torch.float32 and tuple(maximum.shape[1:]) == (H,) and maximum.stride(1) == 1
    assert maximum.shape[0] == state.shape[0] and norm_w.numel() == H * V and norm_w.is_contiguous()
    wp, wf = _param(norm_w)
    lib = library()
    work = torch.empty(lib.pae_matrix_memory_work_floats(T, H, D, V), dtype=torch.float32, device=proj.device)
    _check(lib.pae_matrix_memory_step(
        code_of(proj.dtype), proj.data_ptr(), proj.stride(0), gate.data_ptr(), gate.stride(0), gate_logits.data_ptr(), T, S,
        seq_runs.data_ptr(), slots.data_ptr(), H, D, V, float(gate_cap), state.data_ptr(), state.stride(0),
        maximum.data_ptr(), maximum.stride(0), wp, wf, float(norm_eps), float(floor_eps), work.data_ptr(), out.data_ptr(),
        _stream()))


def embedding_pairs(out: torch.Tensor, table: torch.Tensor, pairs: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                    tok_seq: torch.Tensor, slots: torch.Tensor, last_token: torch.Tensor, scale: float, buckets: int,
                    mul_prev: int, mul_cur: int) -> None:
    """out[t] = scale * table[ids[t]] + pairs[(prev * mul_prev + ids[t] * mul_cur) % buckets] as float32, `prev`
    the token before in the same sequence (the row before in the step, or `last_token[slot]`, int32 [slots],
    which is moved on to each sequence's last token of the step); at position 0 the row `buckets` of `pairs`.
    A sequence's rows must be consecutive in the step and in order."""
    _not_while_recording("embedding_pairs")
    _gpu(out, table, pairs, ids, positions, tok_seq, slots, last_token)
    T, H = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous() and pairs.is_contiguous()
    assert table.dtype == pairs.dtype and table.shape[1] == H and tuple(pairs.shape) == (buckets + 1, H)
    for t in (ids, positions, tok_seq):
        assert t.dtype == torch.int32 and t.numel() == T and t.is_contiguous()
    assert slots.dtype == torch.int32 and slots.is_contiguous()
    assert last_token.dtype == torch.int32 and last_token.dim() == 1 and last_token.is_contiguous()
    _check(library().pae_embedding_pairs(code_of(table.dtype), out.data_ptr(), table.data_ptr(), pairs.data_ptr(),
                                         ids.data_ptr(), positions.data_ptr(), tok_seq.data_ptr(), slots.data_ptr(),
                                         last_token.data_ptr(), T, H, table.shape[0], float(scale), int(buckets),
                                         int(mul_prev), int(mul_cur), _stream()))


MAX_SUM_TERMS = 4


def sum_norm2(residual: torch.Tensor, terms, w1: Optional[torch.Tensor], w2: Optional[torch.Tensor], eps: float,
              out1: Optional[torch.Tensor], out2: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> None:
    """residual += sum of scale * term over `terms` (a list of (tensor, scale): [T, H] in the outputs' type or
    float32, or float32 partial sums [P, T, H] added in order), in float32; then out1 / out2 (either may be None)
    = residual / sqrt(mean(residual^2) + eps) * w1 / w2.  With `rows` (int32) only those rows are produced and
    the residual is left as it is."""
    _not_while_recording("sum_norm2")
    outs = [o for o in (out1, out2) if o is not None]
    _gpu(residual, w1, w2, rows, *outs, *[t for t, _ in terms])
    H = residual.shape[-1]
    assert residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous()
    assert len(terms) <= MAX_SUM_TERMS
    n = residual.shape[0] if rows is None else rows.numel()
    dtype = outs[0].dtype if outs else torch.float32
    for o, w in ((out1, w1), (out2, w2)):
        if o is not None:
            assert o.shape == (n, H) and o.is_contiguous() and o.dtype == dtype and w is not None and w.numel() == H
    if rows is not None:
        assert rows.dtype == torch.int32 and rows.is_contiguous()
    count = len(terms)
    ptrs = (c_void_p * MAX_SUM_TERMS)()
    is_f32, parts = (c_int * MAX_SUM_TERMS)(), (c_int * MAX_SUM_TERMS)()
    strides, scales = (c_int64 * MAX_SUM_TERMS)(), (c_float * MAX_SUM_TERMS)()
    for j, (t, scale) in enumerate(terms):
        assert t.is_contiguous() and tuple(t.shape[-2:]) == tuple(residual.shape)
        if t.dim() == 3:
            assert t.dtype == torch.float32
        else:
            assert t.dim() == 2 and t.dtype in (torch.float32, dtype)
        ptrs[j], is_f32[j] = t.data_ptr(), 1 if t.dtype == torch.float32 else 0
        parts[j], strides[j], scales[j] = (t.shape[0] if t.dim() == 3 else 1), residual.numel(), float(scale)
    p1, f1 = _param(w1)
    p2, f2 = _param(w2)
    _check(library().pae_sum_norm2(code_of(dtype), residual.data_ptr(), count, ptrs, is_f32, parts, strides, scales, p1, f1,
                                   p2, f2, float(eps), _ptr(rows), _ptr(out1), _ptr(out2), n, H, 1, _stream()))


def norm_join(residual: torch.Tensor, terms, w_out: Optional[torch.Tensor], eps: float,
              w_next: Optional[torch.Tensor] = None, eps_next: float = 0.0, normed: Optional[torch.Tensor] = None,
              rows: Optional[torch.Tensor] = None) -> None:
    """A sublayer's output joins the stream through the norm after it: y = sum of scale * term over `terms` (as for
    `sum_norm2`), residual += y / sqrt(mean(y^2) + eps) * w_out (`w_out` None: residual += y), all float32.  Then,
    as asked: `normed` = residual / sqrt(mean(residual^2) + eps_next) * w_next, the norm before the next sublayer,
    and `rows` = the new residual itself, both in the activation type."""
    _not_while_recording("norm_join")
    outs = [o for o in (normed, rows) if o is not None]
    _gpu(residual, w_out, w_next, *outs, *[t for t, _ in terms])
    T, H = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    assert len(terms) <= MAX_SUM_TERMS
    dtype = outs[0].dtype if outs else None
    for o in outs:
        assert o.shape == (T, H) and o.is_contiguous() and o.dtype == dtype
    assert normed is None or (w_next is not None and w_next.numel() == H)
    assert w_out is None or w_out.numel() == H
    ptrs = (c_void_p * MAX_SUM_TERMS)()
    is_f32, parts = (c_int * MAX_SUM_TERMS)(), (c_int * MAX_SUM_TERMS)()
    strides, scales = (c_int64 * MAX_SUM_TERMS)(), (c_float * MAX_SUM_TERMS)()
    for j, (t, scale) in enumerate(terms):
        assert t.is_contiguous() and tuple(t.shape[-2:]) == (T, H)
        if t.dim() == 3:
            assert t.dtype == torch.float32
        else:
            assert t.dim() == 2
            if t.dtype != torch.float32:
                assert dtype is None or t.dtype == dtype
                dtype = t.dtype
        ptrs[j], is_f32[j] = t.data_ptr(), 1 if t.dtype == torch.float32 else 0
        parts[j], strides[j], scales[j] = (t.shape[0] if t.dim() == 3 else 1), residual.numel(), float(scale)
    po, fo = _param(w_out)
    pn, fn = _param(w_next)
    _check(library().pae_norm_join(code_of(dtype or torch.float32), residual.data_ptr(), len(terms), ptrs, is_f32, parts,
                                   strides, scales, po, fo, float(eps), pn, fn, float(eps_next), _ptr(normed), _ptr(rows),
                                   T, H, _stream()))


def linear_attention_step(proj: torch.Tensor, decay_in: torch.Tensor, decay_bias: Optional[torch.Tensor], tau: float,
                          gate: torch.Tensor, out: torch.Tensor, seq_runs: torch.Tensor, slots: torch.Tensor,
                          state: torch.Tensor, norm_w: torch.Tensor, H: int, D: int, V: int, norm_eps: float,
                          gate_activation: str = "silu") -> None:
    """Gated linear attention over a step's rows.  `proj` [T, >= 2HD + HV] holds per token [q | k | v]; `decay_in`
    [T, HD] and `gate` [T, HV] are views of rows in proj's type; `decay_bias` [HD] joins the decay's input in float32,
    and the decay is sigmoid(.)^(1 / tau) per head and key channel.  `seq_runs` int32 [S, 4] = (first row, rows, tokens
    before, 0) per sequence; `slots` int32 [S]; `state` float32 [slots, H, V, D] is the requests' state, read and
    moved on; `out` [T, H * V] receives the read-out, normed over V with `norm_w` [V] and gated, in proj's type."""
    _not_while_recording("linear_attention_step")
    _gpu(proj, decay_in, decay_bias, gate, out, seq_runs, slots, state, norm_w)
    T, S = proj.shape[0], seq_runs.shape[0]
    assert gate_activation in ("silu", "sigmoid")
    assert proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= 2 * H * D + H * V
    for view, width in ((decay_in, H * D), (gate, H * V)):
        assert view.dim() == 2 and view.shape == (T, width) and view.dtype == proj.dtype and view.stride(1) == 1
    assert out.shape == (T, H * V) and out.is_contiguous() and out.dtype == proj.dtype
    assert slots.dtype == torch.int32 and slots.numel() >= S and slots.is_contiguous()
    assert seq_runs.dtype == torch.int32 and seq_runs.shape == (S, 4) and seq_runs.is_contiguous()
    assert seq_runs.data_ptr() % 16 == 0
    assert state.dtype == torch.float32 and tuple(state.shape[1:]) == (H, V, D) and state[0].is_contiguous()
    assert norm_w.numel() == V and norm_w.is_contiguous()
    if decay_bias is not None:
        assert decay_bias.numel() == H * D and decay_bias.is_contiguous()
    wp, wf = _param(norm_w)
    bp, bf = _param(decay_bias)
    lib = library()
    work = torch.empty(lib.pae_linear_attention_work_floats(T, H, D, V), dtype=torch.float32, device=proj.device)
    _check(lib.pae_linear_attention_step(
        code_of(proj.dtype), proj.data_ptr(), proj.stride(0), decay_in.data_ptr(), decay_in.stride(0), bp, bf, float(tau),
        gate.data_ptr(), gate.stride(0), 1 if gate_activation == "sigmoid" else 0, T, S, seq_runs.data_ptr(),
        slots.data_ptr(), H, D, V, state.data_ptr(), state.stride(0), wp, wf, float(norm_eps), work.data_ptr(),
        out.data_ptr(), _stream()))


def project_f32(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [M, N] = a [M, K] w[N, K]^T (+ bias), summed in float32 from operands of either type: for the few
    output features whose sums must not pass the activation type (router and gate logits)."""
    _not_while_recording("project_f32")
    _gpu(a, w, bias)
    M, K = a.shape
    assert a.dim() == 2 and a.stride(1) == 1 and w.dim() == 2 and w.is_contiguous() and w.shape[1] == K and w.dtype == a.dtype
    out = torch.empty((M, w.shape[0]), dtype=torch.float32, device=a.device)
    bp, bf = _param(bias)
    if bias is not None:
        assert bias.numel() == w.shape[0] and bias.is_contiguous()
    _check(library().pae_project_f32(code_of(a.dtype), out.data_ptr(), out.stride(0), a.data_ptr(), a.stride(0),
                                     w.data_ptr(), bp, bf, M, w.shape[0], K, _stream()))
    return out


def moe_route(logits: torch.Tensor, groups: int, keep: int, top: int, scale: float,
              choice_bias: Optional[torch.Tensor] = None):
    """(chosen int32 [T, top], weights float32 [T, top]) from router logits float32 [T, E]: scores are the softmax
    over all experts; only experts of the `keep` best of `groups` equal groups of neighbours (a group's score is
    its largest) can be chosen; the weights are the chosen scores times `scale`.  With `choice_bias` (float32 [E])
    experts and groups are compared by score + bias; the weights stay the scores."""
    _not_while_recording("moe_route")
    _gpu(logits, choice_bias)
    T, E = logits.shape
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    if choice_bias is not None:
        assert choice_bias.dtype == torch.float32 and choice_bias.numel() == E and choice_bias.is_contiguous()
    chosen = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _check(library().pae_moe_route(logits.data_ptr(), T, E, int(groups), int(keep), int(top), float(scale),
                                   _ptr(choice_bias), chosen.data_ptr(), weights.data_ptr(), _stream()))
    return chosen, weights


def moe_experts(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor, chosen: torch.Tensor,
                weights: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """For every token the weighted sum over its chosen experts of W_down[e] (act(W_gate[e] x) * (W_up[e] x));
    `gate_w`, `up_w` [E, F, H] and `down_w` [E, H, F] in x's type.  Returns float32 [T, H], or, from the
    matrix-core kernels (bfloat16, widths in multiples of 32), float32 [top, T, H] whose `top` parts add up to it."""
    _not_while_recording("moe_experts")
    _gpu(x, gate_w, up_w, down_w, chosen, weights)
    T, H = x.shape
    E, F, _ = gate_w.shape
    top = chosen.shape[1]
    assert x.stride(1) == 1 and gate_w.shape == up_w.shape == (E, F, H) and down_w.shape == (E, H, F)
    for w in (gate_w, up_w, down_w):
        assert w.is_contiguous() and w.dtype == x.dtype
    assert chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.shape[0] == T
    assert weights.dtype == torch.float32 and weights.shape == chosen.shape and weights.is_contiguous()
    assert activation in ACTIVATIONS
    act = torch.empty((T * top, F), dtype=x.dtype, device=x.device)
    lib = library()
    if x.dtype == torch.bfloat16 and lib.pae_moe_tiles_supported(H, F) and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0:
        parts = torch.empty((top, T, H), dtype=torch.float32, device=x.device)
        order = torch.empty(T * top, dtype=torch.int32, device=x.device)
        tiles = torch.empty((lib.pae_moe_max_tiles(T * top, E), 4), dtype=torch.int32, device=x.device)
        _check(lib.pae_moe_experts_tiles(parts.data_ptr(), x.data_ptr(), x.stride(0), gate_w.data_ptr(), up_w.data_ptr(),
                                         down_w.data_ptr(), chosen.data_ptr(), weights.data_ptr(), T, top, E, H, F,
                                         ACTIVATIONS[activation], order.data_ptr(), tiles.data_ptr(), act.data_ptr(),
                                         _stream()))
        return parts
    out = torch.empty((T, H), dtype=torch.float32, device=x.device)
    _check(lib.pae_moe_gate_up(code_of(x.dtype), act.data_ptr(), x.data_ptr(), x.stride(0), gate_w.data_ptr(),
                               up_w.data_ptr(), chosen.data_ptr(), T, top, H, F, ACTIVATIONS[activation], _stream()))
    _check(lib.pae_moe_down(code_of(x.dtype), out.data_ptr(), act.data_ptr(), down_w.data_ptr(), chosen.data_ptr(),
                            weights.data_ptr(), T, top, H, F, _stream()))
    return out


def _check_bias_operands(slopes, gate, nh: int, hd: int, q: torch.Tensor):
    """(gate pointer, gate row stride) after checking the slopes and the gate rows of a biased attention call."""
    if slopes is not None:
        assert slopes.dtype == torch.float32 and slopes.numel() == nh and slopes.is_contiguous()
    if gate is None:
        return None, 0
    assert gate.dim() == 2 and gate.shape[0] == q.shape[0] and gate.stride(1) == 1 and gate.shape[1] >= nh * hd
    assert gate.dtype == torch.bfloat16
    return gate.data_ptr(), gate.stride(0)


def mfma_attention_supported(dtype: torch.dtype, nh: int, nkv: int, hd: int, bs: int) -> bool:
    """Shapes the matrix-core attention kernels take; others go through the generic kernel."""
    return dtype == torch.bfloat16 and hd % 32 == 0 and 32 <= hd <= 256 and bs % 16 == 0 and nh // nkv <= 16


def attn_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                dec_work: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                window: int, softcap: float = 0.0, sinks: Optional[torch.Tensor] = None, chunked: bool = False,
                slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> None:
    """Attention of the single new token of each sequence listed in `dec_work` over that sequence's
    cached keys: split over the keys, then merged.  dec_work[i] = (flat row of the token, its
    position, row of its sequence in `block_tables`, 0).  `softcap` > 0 caps the scores
    (s <- softcap tanh(s / softcap)); `sinks` (float32 [nh]) join each head's softmax denominator.
    `chunked`, `slopes`, `gate`: as in `paged_attention_masked` (not together with a cap or sinks)."""
    _gpu(out, q, k_cache, v_cache, dec_work, block_tables, sinks, slopes, gate)
    wide = bool(softcap) or sinks is not None
    biased = chunked or slopes is not None or gate is not None
    assert not (wide and biased)
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == nh and sinks.is_contiguous()
    bs = k_cache.shape[2]
    assert q.dtype == torch.bfloat16 == out.dtype == k_cache.dtype and q.stride(1) == 1 and out.stride(1) == 1
    assert q.shape[1] >= nh * hd and out.shape[1] >= nh * hd and out.shape[0] == q.shape[0]
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert dec_work.dtype == torch.int32 and dec_work.dim() == 2 and dec_work.shape[1] == 4 and dec_work.is_contiguous()
    assert dec_work.data_ptr() % 16 == 0, "the decode work list must start on a 16-byte boundary"
    n = dec_work.shape[0]
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    # (the kernel looks at row i of the tables before it knows token i's own row: the rows must be there)
    assert n <= block_tables.shape[0], "more single tokens than sequences in the tables"
    max_splits = -(-block_tables.shape[1] * bs // library().pae_attn_decode_split())
    part_acc = torch.empty((n * nh * max_splits, hd), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((n * nh * max_splits, 2), dtype=torch.float32, device=q.device)
    if biased:
        _not_while_recording("attn_decode with chunks, a bias by distance or a gate")
        gp, gs = _check_bias_operands(slopes, gate, nh, hd, q)
        _check(library().pae_attn_decode_biased_bf16(
            out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
            dec_work.data_ptr(), n, block_tables.data_ptr(), block_tables.shape[1], bs, nh, nkv, hd, float(scale),
            int(window), 1 if chunked else 0, _ptr(slopes), gp, gs, part_acc.data_ptr(), part_ml.data_ptr(), _stream()))
        return
    if wide:
        _not_while_recording("attn_decode with a score cap or sinks")
        _check(library().pae_attn_decode_capped_bf16(
            out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
            dec_work.data_ptr(), n, block_tables.data_ptr(), block_tables.shape[1], bs, nh, nkv, hd, float(scale),
            int(window), float(softcap), _ptr(sinks), part_acc.data_ptr(), part_ml.data_ptr(), _stream()))
        return
    if _RECORDING is not None:
        _RECORDING.room(2)  # the splits' partial results, then their merge
        code = library().pae_program_put_attention(
            _RECORDING.host_ptr, _RECORDING.count, out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0),
            k_cache.data_ptr(), v_cache.data_ptr(), dec_work.data_ptr(), n, block_tables.data_ptr(),
            block_tables.shape[1], bs, nh, nkv, hd, float(scale), int(window), part_acc.data_ptr(), part_ml.data_ptr())
        _RECORDING.add(code, out, q, part_acc, part_ml)
        _RECORDING.add(code)
        return
    _check(library().pae_attn_decode_bf16(
        out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        dec_work.data_ptr(), n, block_tables.data_ptr(), block_tables.shape[1], bs, nh, nkv, hd, float(scale),
        int(window), part_acc.data_ptr(), part_ml.data_ptr(), _stream()))


PREFILL_TILE = 64  # tokens per run of the prefill attention kernel (one workgroup each)


def attn_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 tiles: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor,
                 nh: int, nkv: int, hd: int, scale: float, window: int, softcap: float = 0.0,
                 sinks: Optional[torch.Tensor] = None, chunked: bool = False, slopes: Optional[torch.Tensor] = None,
                 gate: Optional[torch.Tensor] = None) -> None:
    """Attention of runs of consecutive tokens; tiles[t] = (table row of the sequence, first
    flat token, number of tokens <= PREFILL_TILE).  One workgroup per run and head, whose
    wavefronts share out the keys; workgroups start in the order of `tiles`, so the runs with
    the most keys should come first.  `softcap`, `sinks`, `chunked`, `slopes` and `gate` as in `attn_decode`."""
    _not_while_recording("attn_prefill")
    _gpu(out, q, k_cache, v_cache, tiles, positions, block_tables, sinks, slopes, gate)
    biased = chunked or slopes is not None or gate is not None
    assert not (biased and (softcap or sinks is not None))
    if sinks is not None:
        assert sinks.dtype == torch.float32 and sinks.numel() == nh and sinks.is_contiguous()
    bs = k_cache.shape[2]
    assert q.dtype == torch.bfloat16 == out.dtype == k_cache.dtype and q.stride(1) == 1 and out.stride(1) == 1
    assert q.shape[1] >= nh * hd and out.shape[1] >= nh * hd and out.shape[0] == q.shape[0]
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 3 and tiles.is_contiguous()
    assert positions.dtype == torch.int32 and positions.numel() == q.shape[0]
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    if biased:
        gp, gs = _check_bias_operands(slopes, gate, nh, hd, q)
        _check(library().pae_attn_prefill_biased_bf16(
            out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
            tiles.data_ptr(), tiles.shape[0], positions.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
            bs, nh, nkv, hd, float(scale), int(window), 1 if chunked else 0, _ptr(slopes), gp, gs, _stream()))
        return
    _check(library().pae_attn_prefill_capped_bf16(
        out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        tiles.data_ptr(), tiles.shape[0], positions.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
        bs, nh, nkv, hd, float(scale), int(window), float(softcap), _ptr(sinks), _stream()))


def sample(tokens: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor],
           uniform: Optional[torch.Tensor]) -> None:
    """tokens[r] = argmax(logits[r]) where temperature[r] == 0 (or no temperatures
    are given), else the inverse-CDF sample of softmax(logits[r] / temperature[r]) at uniform[r]."""
    _not_while_recording("sample")
    _gpu(tokens, logits, temperature, uniform)
    R, V = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert tokens.dtype == torch.int32 and tokens.numel() == R
    for t in (temperature, uniform):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == R
    chunks = library().pae_sample_chunks(V)
    chunk_max = torch.empty(R * chunks, dtype=torch.float32, device=logits.device)
    chunk_arg = torch.empty(R * chunks, dtype=torch.int32, device=logits.device)
    chunk_sum = (torch.empty(R * chunks, dtype=torch.float64, device=logits.device)
                 if temperature is not None else None)
    _check(library().pae_sample(tokens.data_ptr(), logits.data_ptr(), logits.stride(0), _ptr(temperature),
                                _ptr(uniform), R, V, chunk_max.data_ptr(), chunk_arg.data_ptr(),
                                _ptr(chunk_sum), _stream()))


def sample_static(tokens: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor],
                  uniform: Optional[torch.Tensor]) -> None:
    """`sample` without a workspace: the chunk results go to a buffer inside the library's image on
    the GPU, so nothing is allocated here or there.  Rows times chunks beyond that buffer's slots
    are refused; calls that overlap on one GPU race (they share the buffer)."""
    _not_while_recording("sample_static")
    _gpu(tokens, logits, temperature, uniform)
    R, V = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert tokens.dtype == torch.int32 and tokens.numel() == R
    for t in (temperature, uniform):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == R
    _check(library().pae_sample_static(tokens.data_ptr(), logits.data_ptr(), logits.stride(0), _ptr(temperature),
                                       _ptr(uniform), R, V, _stream()))
