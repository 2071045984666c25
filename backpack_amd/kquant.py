"""Host-side op layer over the C ABI, with torch tensors as device memory.

Mirrors the reference's k-quant operator shape: a packed weight descriptor
(KQuantPacked: data, N, K, rowStrideWords, nBlocks — runtime/gguf_loader.h:108-113)
and a matmul taking the {X, W, Bias, Y, P} binding set
(runtime/model_runner.cpp:2404-2413).  torch only owns the buffers and the
stream; every computation goes through libbpk_kquant.so.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from . import capi
from .capi import Q4_K, Q5_K, Q6_K  # noqa: F401


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


@dataclass
class KQuantPacked:
    """Packed k-quant matrix resident on the GPU (same fields as the reference's)."""
    data: torch.Tensor        # uint8, N * row_stride_words * 4 bytes (+16 slack)
    type: int
    N: int
    K: int
    row_stride_words: int
    n_blocks: int

    @property
    def row_stride_bytes(self) -> int:
        return self.row_stride_words * 4


def pack_host(type_: int, raw: np.ndarray, N: int, K: int) -> np.ndarray:
    """pack_q4k / pack_q6k on the host through the library's packer."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    nb, rs = capi.layout(type_, K)
    assert raw.size == N * nb * {12: 144, 13: 176, 14: 210}[type_], "raw size does not match N x K"
    out = np.empty(N * rs, dtype=np.uint32)
    capi.check(capi.lib().bpk_kq_pack_host(type_, raw.ctypes.data, N, K, out.ctypes.data))
    return out


def upload(type_: int, packed_words: np.ndarray, N: int, K: int, device="cuda") -> KQuantPacked:
    """Packed host words -> device (the reference's uploadKQWeight)."""
    nb, rs = capi.layout(type_, K)
    assert packed_words.size == N * rs
    host = torch.from_numpy(np.ascontiguousarray(packed_words).view(np.uint8))
    data = torch.zeros(host.numel() + 16, dtype=torch.uint8, device=device)
    data[: host.numel()].copy_(host)
    return KQuantPacked(data, type_, N, K, rs, nb)


def from_raw(type_: int, raw: np.ndarray, N: int, K: int, device="cuda") -> KQuantPacked:
    return upload(type_, pack_host(type_, raw, N, K), N, K, device)


class _LibraryWeight:
    """Device allocation owned by the library (bpk_weight); freed with the object."""

    def __init__(self, handle, desc):
        self._h, self._ptr, self.nbytes = handle, desc.data, desc.bytes
        self.device = torch.device("cuda", torch.cuda.current_device())

    def data_ptr(self) -> int:
        return self._ptr

    def __del__(self):
        try:
            if self._h:
                capi.lib().bpk_weight_destroy(self._h)
                self._h = None
        except Exception:
            pass


def from_gguf(g, names) -> KQuantPacked:
    """Named Q4_K / Q6_K tensors of an open GGUFFile -> one device weight, rows stacked in order
    (the loader's tensor -> packKQ -> fuseKQ -> uploadKQWeight, runtime/model_runner.cpp:1275-1338)."""
    import ctypes as C
    names = [names] if isinstance(names, str) else list(names)
    arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
    h = C.c_void_p()
    capi.check(capi.lib().bpk_gguf_weight_create(g.handle, arr, len(names), C.byref(h)))
    d = capi.WeightDesc()
    capi.check(capi.lib().bpk_weight_describe(h, C.byref(d)))
    return KQuantPacked(_LibraryWeight(h, d), d.type, d.N, d.K, d.row_stride_words, d.n_blocks)


def fuse(parts: list[KQuantPacked]) -> KQuantPacked:
    """Row-wise concatenation of matrices with equal K and type (fuseKQ)."""
    a = parts[0]
    assert all(p.K == a.K and p.type == a.type for p in parts)
    body = [p.data[: p.N * p.row_stride_bytes] for p in parts]
    data = torch.cat(body + [torch.zeros(16, dtype=torch.uint8, device=a.data.device)])
    return KQuantPacked(data, a.type, sum(p.N for p in parts), a.K, a.row_stride_words, a.n_blocks)


def matmul(x: torch.Tensor, w: KQuantPacked, bias: torch.Tensor | None = None,
           out: torch.Tensor | None = None, y_offset: int = 0) -> torch.Tensor:
    """Y[m, y_offset+n] = bias[n] + sum_k X[m,k] * dequant(W)[n,k]; fp32 or bf16 X."""
    assert x.is_cuda and x.is_contiguous() and x.shape[-1] == w.K
    M = x.numel() // w.K
    if out is None:
        assert y_offset == 0
        out = torch.empty((M, w.N), dtype=torch.float32, device=x.device)
    assert out.is_contiguous() and out.dtype == torch.float32
    L = capi.lib()
    if x.dtype == torch.float32:
        rc = L.bpk_kq_matmul(w.type, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), M, w.N, w.K,
                             w.n_blocks, w.row_stride_words, y_offset, _stream())
    elif x.dtype == torch.bfloat16:
        assert y_offset == 0
        rc = L.bpk_kq_matmul_bf16(w.type, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), M, w.N, w.K,
                                  w.n_blocks, w.row_stride_words, _stream())
    else:
        raise TypeError(f"X must be float32 or bfloat16, got {x.dtype}")
    capi.check(rc)
    return out


def prefill_rows_bf16(x: torch.Tensor, K: int, prologue: int = capi.PRO_NONE, norm_w: torch.Tensor | None = None,
                      eps: float = 0.0) -> torch.Tensor:
    """fp32 rows -> the bf16 activation rows of the prefill GEMM, [M, K]: x as it is, its RMSNorm, or
    act(gate) * up of gate|up rows of 2K floats, evaluated in fp32 and rounded to nearest even."""
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32
    row = 2 * K if prologue in (capi.PRO_SILU_MUL, capi.PRO_GELU_MUL) else K
    assert x.shape[-1] == row
    M = x.numel() // row
    out = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
    capi.check(capi.lib().bpk_prefill_rows_bf16(prologue, _ptr(x), _ptr(norm_w), eps, M, K, _ptr(out), _stream()))
    return out


def matmul_fused(x: torch.Tensor, w: KQuantPacked, prologue: int = capi.PRO_NONE, norm_w: torch.Tensor | None = None,
                 eps: float = 0.0, residual: torch.Tensor | None = None, bias: torch.Tensor | None = None,
                 out: torch.Tensor | None = None, workspace: torch.Tensor | None = None,
                 allow_workspace: bool = True, epilogue: int = capi.EPI_NONE) -> torch.Tensor:
    """The decode matvec with what surrounds it folded in: RMSNorm of x, or act(gate)*up of a gate|up
    row (x is then [M, 2K]), and a residual added to the output (residual may be `out`).  With an
    epilogue, w is the stacked gate|up matrix and the result is act(gate.x) * (up.x), [M, w.N / 2]."""
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32
    xk = w.K * (2 if prologue in (capi.PRO_SILU_MUL, capi.PRO_GELU_MUL) else 1)
    assert x.shape[-1] == xk
    M = x.numel() // xk
    n_out = w.N // 2 if epilogue else w.N
    if out is None:
        out = torch.empty((M, n_out), dtype=torch.float32, device=x.device)
    L = capi.lib()
    f = capi.Fusion(prologue, _ptr(norm_w), eps, _ptr(residual), epilogue)
    nbytes = 0
    if workspace is None and allow_workspace:
        nbytes = L.bpk_kq_matmul_fused_workspace_bytes(M, n_out, w.K)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    elif workspace is not None:
        nbytes = workspace.numel() * workspace.element_size()
    capi.check(L.bpk_kq_matmul_fused(w.type, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), M, n_out, w.K, w.n_blocks,
                                     w.row_stride_words, 0, f, _ptr(workspace), nbytes, _stream()))
    return out


class Chain:
    """A recorded list of decode matvecs (M = 1) with their fused forms; run(first, count) issues a stretch
    of it as one launch (bpk_chain_*).  Ops are added with the arguments of matmul_fused; an op whose x or
    residual is the output buffer of an earlier op follows that op."""

    def __init__(self):
        self._ops, self._keep, self._h = [], [], None

    def add(self, x, w: KQuantPacked, out, prologue=capi.PRO_NONE, norm_w=None, eps=0.0, residual=None, bias=None,
            epilogue=capi.EPI_NONE, y_offset=0) -> int:
        assert self._h is None, "the chain is already built"
        n_out = w.N // 2 if epilogue else w.N
        op = capi.ChainOp(w.type, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), n_out, w.K, w.n_blocks,
                          w.row_stride_words, y_offset,
                          capi.Fusion(prologue, _ptr(norm_w), eps, _ptr(residual), epilogue))
        self._ops.append(op)
        self._keep.append((x, w, out, norm_w, residual, bias))      # the buffers live as long as the chain
        return len(self._ops) - 1

    def build(self) -> "Chain":
        import ctypes as C
        arr = (capi.ChainOp * len(self._ops))(*self._ops)
        h = C.c_void_p()
        capi.check(capi.lib().bpk_chain_create(arr, len(self._ops), C.byref(h)))
        self._h = h
        return self

    def __len__(self):
        return len(self._ops)

    def run(self, first: int = 0, count: int | None = None) -> None:
        count = len(self._ops) - first if count is None else count
        capi.check(capi.lib().bpk_chain_run(self._h, first, count, _stream()))

    def status(self) -> None:
        capi.check(capi.lib().bpk_chain_status(self._h))

    def reset(self) -> None:
        capi.check(capi.lib().bpk_chain_reset(self._h))

    def __del__(self):
        try:
            if self._h:
                capi.lib().bpk_chain_destroy(self._h)
                self._h = None
        except Exception:
            pass


def argmax_rows(logits: torch.Tensor):
    """(index int32 [M], value f32 [M]) of the largest element of each row; lowest index on ties."""
    assert logits.is_cuda and logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1
    M, N = logits.shape
    idx = torch.empty(M, dtype=torch.int32, device=logits.device)
    val = torch.empty(M, dtype=torch.float32, device=logits.device)
    capi.check(capi.lib().bpk_argmax_rows(_ptr(logits), M, N, logits.stride(0), _ptr(idx), _ptr(val), _stream()))
    return idx, val


def matmul_argmax(x: torch.Tensor, w: KQuantPacked, bias: torch.Tensor | None = None):
    """lm_head and greedy pick in one call: (logits [M,N], index int32 [M], value f32 [M])."""
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float32 and x.shape[-1] == w.K
    M = x.numel() // w.K
    logits = torch.empty((M, w.N), dtype=torch.float32, device=x.device)
    idx = torch.empty(M, dtype=torch.int32, device=x.device)
    val = torch.empty(M, dtype=torch.float32, device=x.device)
    capi.check(capi.lib().bpk_kq_matmul_argmax(w.type, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(logits), M, w.N, w.K,
                                               w.n_blocks, w.row_stride_words, _ptr(idx), _ptr(val), _stream()))
    return logits, idx, val


def dequant_rows(w: KQuantPacked, rows: torch.Tensor | None = None, M: int | None = None) -> torch.Tensor:
    """fp32 rows of the matrix (the q6k_gather contract); rows: int32 device tensor."""
    if rows is not None:
        assert rows.dtype == torch.int32 and rows.is_cuda
        M = rows.numel()
    elif M is None:
        M = w.N
    out = torch.empty((M, w.K), dtype=torch.float32, device=w.data.device)
    capi.check(capi.lib().bpk_kq_dequant_rows(w.type, _ptr(w.data), w.row_stride_words, _ptr(rows), M, w.K,
                                              _ptr(out), _stream()))
    return out


def moe_matmul(x: torch.Tensor, w: KQuantPacked, expert_idx: torch.Tensor, n_experts: int,
               x_per_slot: bool = False) -> torch.Tensor:
    """Per (token, slot) matvec against the expert's row slice of a stacked matrix."""
    assert expert_idx.dtype in (torch.int32, torch.uint32) and expert_idx.is_cuda
    T, k = expert_idx.shape
    N = w.N // n_experts
    assert N * n_experts == w.N
    out = torch.empty((T, k, N), dtype=torch.float32, device=x.device)
    capi.check(capi.lib().bpk_kq_moe_matmul(w.type, _ptr(x), _ptr(w.data), _ptr(expert_idx), _ptr(out), T, k,
                                            n_experts, N, w.K, w.n_blocks, w.row_stride_words,
                                            int(x_per_slot), _stream()))
    return out


def moe_topk_softmax(logits: torch.Tensor, k: int, normalize: bool = True):
    """Router selection per token: (idx int32 [T,k], wt f32 [T,k]) from logits f32 [T, n_experts]."""
    assert logits.is_cuda and logits.is_contiguous() and logits.dtype == torch.float32
    T, E = logits.shape
    idx = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    wt = torch.empty((T, k), dtype=torch.float32, device=logits.device)
    capi.check(capi.lib().bpk_moe_topk_softmax(_ptr(logits), T, E, k, int(normalize), _ptr(idx), _ptr(wt), _stream()))
    return idx, wt


def moe_route(x: torch.Tensor, router_w: torch.Tensor, k: int, normalize: bool = True, want_logits: bool = False):
    """Router matvec (fp32 [n_experts, hidden]) and selection in one launch."""
    assert x.is_contiguous() and router_w.is_contiguous() and x.dtype == router_w.dtype == torch.float32
    T, H = x.shape
    E = router_w.shape[0]
    idx = torch.empty((T, k), dtype=torch.int32, device=x.device)
    wt = torch.empty((T, k), dtype=torch.float32, device=x.device)
    logits = torch.empty((T, E), dtype=torch.float32, device=x.device) if want_logits else None
    capi.check(capi.lib().bpk_moe_route(_ptr(x), _ptr(router_w), T, H, E, k, int(normalize), _ptr(logits), _ptr(idx),
                                        _ptr(wt), _stream()))
    return (idx, wt, logits) if want_logits else (idx, wt)


def moe_ffn(x: torch.Tensor, gate: KQuantPacked, up: KQuantPacked, down: KQuantPacked,
            expert_idx: torch.Tensor, expert_wt: torch.Tensor, n_experts: int) -> torch.Tensor:
    """Routed-expert FFN: sum_s wt[t,s] * down_e(silu(gate_e x) * up_e x)."""
    T, k = expert_idx.shape
    hidden, inter = gate.K, down.K
    L = capi.lib()
    nbytes = L.bpk_kq_moe_ffn_scratch_bytes(T, k, hidden, inter)
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    out = torch.empty((T, hidden), dtype=torch.float32, device=x.device)
    capi.check(L.bpk_kq_moe_ffn(gate.type, down.type, _ptr(x), _ptr(gate.data), _ptr(up.data), _ptr(down.data),
                                _ptr(expert_idx), _ptr(expert_wt), _ptr(out), T, k, n_experts, hidden, inter,
                                _ptr(scratch), nbytes, _stream()))
    return out
