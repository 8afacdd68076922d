"""Host wrappers: drop-in `matmul(a, b)` / `attention(q, k, v, causal, sm_scale)` of the
reference tutorials plus `mx_matmul`, on top of the C ABI.

Mirrors, argument for argument,
  python/tutorials/03-matrix-multiplication.py:330-348   matmul(a, b, activation="")
  python/tutorials/06-fused-attention.py:438-520         _attention / attention
  python/tutorials/09-persistent-matmul.py:105-138       matmul(a, b) with out dtype = in dtype
Tensors may be torch tensors or any object exposing data_ptr(), dtype, shape, stride(i)
and device (the duck typing of the reference launcher, third_party/amd/backend/driver.py:285-323).
"""
from __future__ import annotations

import os

import math

import torch

from . import _lib, hooks

_TORCH_TO_ABI = {
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
    torch.float8_e4m3fn: _lib.F8E4M3,
    torch.float8_e5m2: _lib.F8E5M2,
    torch.float32: _lib.F32,
}
# names the reference uses for reinterpret()-ed tensors (python/triton/runtime/jit.py:406-429)
_NAME_TO_ABI = {
    "fp16": _lib.F16, "bf16": _lib.BF16, "fp8e4nv": _lib.F8E4M3, "fp8e5": _lib.F8E5M2, "fp32": _lib.F32,
    "float16": _lib.F16, "bfloat16": _lib.BF16, "float8_e4m3fn": _lib.F8E4M3, "float8_e5m2": _lib.F8E5M2,
}
_ABI_TO_TORCH = {v: k for k, v in _TORCH_TO_ABI.items()}
_ELEM_BYTES = {_lib.F16: 2, _lib.BF16: 2, _lib.F8E4M3: 1, _lib.F8E5M2: 1, _lib.F32: 4}


def _abi_dtype(t) -> int:
    dt = t.dtype
    if dt in _TORCH_TO_ABI:
        return _TORCH_TO_ABI[dt]
    name = getattr(dt, "name", None) or str(dt)
    name = name.split(".")[-1]
    if name in _NAME_TO_ABI:
        return _NAME_TO_ABI[name]
    raise TypeError(f"unsupported dtype {dt}")


def _check_device(idx: int, t) -> None:
    dev = getattr(t, "device", None)
    if dev is None and hasattr(t, "base"):
        dev = getattr(t.base, "device", None)
    if dev is not None and getattr(dev, "type", "cuda") != "cuda":
        raise ValueError(f"Pointer argument (at {idx}) cannot be accessed from Triton (cpu tensor?)")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _is_contiguous(t) -> bool:
    if hasattr(t, "is_contiguous"):
        return t.is_contiguous()
    expect = 1
    for d in range(len(t.shape) - 1, -1, -1):
        if t.shape[d] != 1 and t.stride(d) != expect:
            return False
        expect *= t.shape[d]
    return True


_scale_cache = {}


def _scale_ptr(s, device):
    """None, a python float or a 1-element fp32 device tensor -> (pointer or None, keep-alive).
    A python float becomes a device scalar once per (device, value): repeated calls with the same
    scale pay no host-to-device copy."""
    if s is None:
        return None, None
    if not isinstance(s, torch.Tensor):
        key = (str(device), float(s))
        t = _scale_cache.get(key)
        if t is None:
            if len(_scale_cache) >= 256:
                _scale_cache.clear()
            t = _scale_cache[key] = torch.tensor([float(s)], dtype=torch.float32, device=device)
        s = t
    assert s.dtype == torch.float32 and s.numel() == 1, "scales are one fp32 value per tensor"
    _check_device(-1, s)
    return s.data_ptr(), s


_cu_count = {}   # device index -> compute units


def _splitk_splits(device, M, N, k_bytes, fp32=False):
    """Number of K splits for `matmul` (0 = none): products with less than half a round of 128x128 tiles and a long K
    give every tile to several workgroups (`mi355_gemm_splitk`) - one workgroup per CU, at least sixteen 64-byte K steps
    each, at most 32 slices and 64 MiB of fp32 partial sums.  Shapes with at most 64 rows on a side (and up to 128
    against a long other side) stay with the streaming kernels."""
    if os.environ.get("MI355_GEMM_SPLITK", "1") == "0":
        return 0
    small, large = min(M, N), max(M, N)
    if small <= 64 or (small <= 128 and large >= 2048):
        return 0
    idx = device.index if device.index is not None else torch.cuda.current_device()
    cus = _cu_count.get(idx)
    if cus is None:
        cus = _cu_count[idx] = max(1, _lib.load().mi355_query(_lib.Q_CU_COUNT))
    tiles = -(-M // 128) * -(-N // 128)
    ksteps = -(-k_bytes // 64)
    if fp32:
        # bound by the fp32 MFMA rate alone: whatever puts more CUs to work wins, down to eight K steps a slice (two
        # workgroups per CU; flushed do_bench, 1024^3: 74 -> 24 us)
        if tiles >= cus or ksteps < 16:
            return 0
        splits = min(-(-2 * cus // tiles), ksteps // 8, 32, (64 << 20) // (4 * M * N))
        return splits if splits >= 2 else 0
    if tiles * 2 > cus or ksteps < 64:
        return 0
    # one workgroup per CU, at least 16 K steps each (flushed do_bench, bf16, us by number of splits - 1 / 2 / 4 / 8 / 16 /
    # 32: 256 x 256 x 4096 51 / 34 / 24 / 20 / 19 / 23, 1024 x 1024 x 4096 52 / 38 / 30 / 36 / 49 / 71, 256 x 8192 x 8192 117 / 81 / 89 /
    # 99 / 122 / 189, 256 x 1024 x 8192 97 / 59 / 39 / 28 / 27 / 35; 1024^3, 32 steps: 18 / 21 / 23 - not split)
    splits = min(cus // tiles, ksteps // 16, 32, (64 << 20) // (4 * M * N))
    return splits if splits >= 2 else 0


def matmul(a, b, activation="", *, out_dtype=None, a_scale=None, b_scale=None, add=None, softmax=False):
    """C = softmax_rows?(act((a_scale*b_scale) * A @ B + add)) with fp32 accumulation.

    Same contract as the reference wrapper (03:330-348): A must be contiguous, B may have any
    strides (the reference passes `b.T` for fp8, 03:378-382), the result is fp16 for fp16 / fp8
    inputs.  Extensions, all keyword-only and defaulting to the reference behaviour: bf16
    inputs give a bf16 result, fp32 inputs (exact fp32 products on the fp32 MFMAs, the `ieee` precision of `tl.dot`) an
    fp16 one like the reference's `c = accumulator.to(tl.float16)`, `out_dtype` overrides the result type, `a_scale` / `b_scale`
    are per-tensor fp32 dequantisation scales; `add` (fp16 / bf16 / fp32, broadcastable to
    [M, N]: a matrix, an [M, 1] column = the reference's add-rows, a [1, N] / [N] row = its
    add-cols) and `softmax` are the fused epilogues of the reference's dot test
    (python/test/unit/language/test_core.py:3128-3141).
    """
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert _is_contiguous(a), "Matrix A must be contiguous"
    in_dt = _abi_dtype(a)
    assert in_dt == _abi_dtype(b), "Incompatible dtypes"
    _check_device(0, a)
    _check_device(1, b)
    M, K = a.shape
    K, N = b.shape
    K_caller = K
    if out_dtype is None:
        out_dtype = torch.bfloat16 if in_dt == _lib.BF16 else torch.float16
    if activation not in ("", "leaky_relu"):
        raise KeyError(f"unknown ACTIVATION {activation!r}")
    device = a.device if isinstance(a, torch.Tensor) else torch.device("cuda", torch.cuda.current_device())
    c = torch.empty((M, N), device=device, dtype=out_dtype)
    if M == 0 or N == 0:
        return c
    if K == 0:
        return c.zero_()
    if (in_dt != _lib.F32 and (K * _ELEM_BYTES[in_dt]) % 16 != 0 and M * N * K >= 1 << 30
            and isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)):
        # Rows of A that are not a multiple of 16 bytes long do not start on 16-byte boundaries, which every MFMA
        # kernel's loads need: the C ABI then runs its strided kernel (4096 x 4096 x 4100 bf16: 43 TFLOP/s).  The
        # reference masks the K tail to zero (03:297-298); appending those zeros to K here - one copy of each
        # operand - gives the same sums on the fast kernels (the same shape: 1000 TFLOP/s).  Below about 2^30
        # multiply-adds the any-stride MFMA kernel is as fast or faster than the copies plus the tile kernels (flushed
        # do_bench, bf16, that kernel / padded: 2048 x 100 x 100 12 / 27 us, 2047 x 257 x 257 16 / 32, 1024 x 1024 x 1000 23 / 23,
        # 1024 x 1024 x 4100 107 / 70).
        pad = -K % (16 // _ELEM_BYTES[in_dt])
        as_bytes = (lambda t: t.view(torch.uint8)) if _ELEM_BYTES[in_dt] == 1 else (lambda t: t)
        a = torch.nn.functional.pad(as_bytes(a), (0, pad)).view(a.dtype)
        if b.stride(0) == 1 and b.stride(1) != 1:      # K-major B: its K axis is the contiguous one of b.t()
            b = torch.nn.functional.pad(as_bytes(b.t()), (0, pad)).view(b.dtype).t()
        else:
            b = torch.nn.functional.pad(as_bytes(b), (0, 0, 0, pad)).view(b.dtype)
        K += pad        # (the launch metadata below keeps the caller's K)
    if (in_dt == _lib.F32 and isinstance(b, torch.Tensor) and b.stride(0) != 1 and K % 4 == 0 and M * N * K >= 1 << 24):
        # fp32 operands run on the fp32 MFMAs with a K-major B only (the LDS transpose reads stop at 16-bit elements): a
        # row-major B is put K-major first - one transposing copy, 1 / M of the product's work -; small products and a K
        # that is not a multiple of four elements take the any-stride kernel of the C ABI as they are
        b = b.t().contiguous().t()
    vec = 16 // _ELEM_BYTES[in_dt] if in_dt != _lib.F32 else 0
    if (vec and isinstance(b, torch.Tensor) and b.stride(1) == 1 and b.stride(0) != 1
            and (b.stride(0) % vec != 0 or b.data_ptr() % 16 != 0) and K % vec == 0 and M * N * K >= 1 << 30):
        # A row-major B runs on the MFMAs inside the C ABI when its rows START on 16-byte boundaries (N itself need not
        # be a multiple: the last chunk of a row then reaches into the padding that the pitch provides).  One whose
        # pitch is not a multiple of 16 bytes would take the any-stride kernel (8100 x 8100 x 8192 bf16: 48 TFLOP/s on
        # the old kernel of that path): its rows are copied into a buffer with a padded pitch first - one plain copy,
        # as the reference spends one on its fp8 case ("pre-transpose b for efficiency", 03:378-380).
        as_bytes = (lambda t: t.view(torch.uint8)) if _ELEM_BYTES[in_dt] == 1 else (lambda t: t)
        b = torch.nn.functional.pad(as_bytes(b), (0, -N % vec)).view(b.dtype)[:, :N]
    pa, keep_a = _scale_ptr(a_scale, device)
    pb, keep_b = _scale_ptr(b_scale, device)
    act = _lib.ACT_LEAKY_RELU if activation == "leaky_relu" else _lib.ACT_NONE
    stream = _stream()
    md = hooks.enter("mi355_gemm", stream, hooks.matmul_launch_metadata, ("mi355_gemm", M, N, K_caller, _ELEM_BYTES[in_dt]))
    if (add is None and not softmax and isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)
            and (in_dt != _lib.F32 or (b.stride(0) == 1 and K % 4 == 0))):
        splits = _splitk_splits(device, M, N, K * _ELEM_BYTES[in_dt], in_dt == _lib.F32)
        if splits:
            # few tiles, long K: every tile's K range is shared out (the fp32 partial sums live in a buffer from
            # torch's caching allocator, which orders its reuse on this stream)
            ws = torch.empty(splits * M * N, dtype=torch.float32, device=device)
            rc = _lib.load().mi355_gemm_splitk(
                a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
                a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                in_dt, _TORCH_TO_ABI[out_dtype], pa, pb, act, splits, ws.data_ptr(), ws.numel() * 4, stream)
            _lib.check(rc, "mi355_gemm_splitk")
            hooks.exit(md)
            return c
    ext = _lib.ext()
    if ext is not None and isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor):
        # the PyTorch-ROCm extension: tensors in, torch's current stream taken in C++, one C-ABI call
        d = None
        if add is not None:
            if add.dtype not in (torch.float16, torch.bfloat16, torch.float32):
                raise TypeError(f"add must be fp16, bf16 or fp32, got {add.dtype}")
            d = torch.broadcast_to(add, (M, N))
        ext.gemm(a, b, c, act, keep_a, keep_b, d, bool(softmax))
        hooks.exit(md)
        return c
    if add is None and not softmax:
        rc = _lib.load().mi355_gemm(
            a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
            a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
            in_dt, _TORCH_TO_ABI[out_dtype], pa, pb, act, stream)
        _lib.check(rc, "mi355_gemm")
        hooks.exit(md)
        return c
    d_ptr, d_sm, d_sn, d_dt = 0, 0, 0, 0
    if add is not None:
        _check_device(2, add)
        if add.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            raise TypeError(f"add must be fp16, bf16 or fp32, got {add.dtype}")
        d = torch.broadcast_to(add, (M, N))  # zero strides on broadcast axes
        d_ptr, d_sm, d_sn, d_dt = d.data_ptr(), d.stride(0), d.stride(1), _TORCH_TO_ABI[add.dtype]
    rc = _lib.load().mi355_gemm_epilogue(
        a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
        a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
        in_dt, _TORCH_TO_ABI[out_dtype], pa, pb, d_ptr, d_sm, d_sn, d_dt, act, int(bool(softmax)), stream)
    _lib.check(rc, "mi355_gemm_epilogue")
    hooks.exit(md)
    return c


_streamk_workspace = {}   # device -> [workspace tensor, stream handle of its last user, event recorded behind that launch]


def _streamk_workspace_for(device, stream, nbytes):
    """ONE partial-tile workspace per device (128 MiB on an MI355X), however many streams call: a call on another
    stream than the previous user's first waits (on the device) for the event recorded behind that launch, so
    launches that share the slots never overlap."""
    entry = _streamk_workspace.get(device)
    if entry is None or entry[0].numel() < nbytes:
        entry = _streamk_workspace[device] = [torch.empty(nbytes, device=device, dtype=torch.uint8), stream, None]
    if entry[1] != stream and entry[2] is not None:
        torch.cuda.current_stream(device).wait_event(entry[2])
    entry[1] = stream
    return entry



def matmul_streamk(a, b, *, out_dtype=None):
    """`matmul(a, b)` with the stream-K schedule: one program per CU, all K steps of all 256x256
    tiles dealt evenly, so tile counts that are not a multiple of the CU count - or smaller than it,
    where this becomes split-K - keep every CU busy.  The scheduling idea of the persistent
    tutorial (python/tutorials/09-persistent-matmul.py:141-190) taken one step further; the
    result is the same `a @ b` (partial tiles are added in a fixed order).  One fp32 workspace per device is
    allocated on first use and kept; calls on different streams are ordered behind one another by an event."""
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert _is_contiguous(a), "Matrix A must be contiguous"
    in_dt = _abi_dtype(a)
    assert in_dt == _abi_dtype(b), "Incompatible dtypes"
    _check_device(0, a)
    _check_device(1, b)
    M, K = a.shape
    _, N = b.shape
    if out_dtype is None:
        out_dtype = torch.bfloat16 if in_dt == _lib.BF16 else torch.float16
    c = torch.empty((M, N), device=a.device, dtype=out_dtype)
    if M == 0 or N == 0:
        return c
    if K == 0:
        return c.zero_()
    lib = _lib.load()
    stream = _stream()
    entry = _streamk_workspace_for(a.device, stream, lib.mi355_query(_lib.Q_STREAMK_WORKSPACE_BYTES))
    ws = entry[0]
    rc = lib.mi355_gemm_streamk(
        a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
        a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
        in_dt, _TORCH_TO_ABI[out_dtype], 0, 0, _lib.ACT_NONE, ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc, "mi355_gemm_streamk")
    if entry[2] is None:
        entry[2] = torch.cuda.Event()
    entry[2].record(torch.cuda.current_stream(a.device))
    return c


def chain_dot(a, b, w, *, out_dtype=None, add=None, activation="", softmax=False):
    """(A @ B [+ add, activation, row softmax]) rounded to the input type, then @ W: the CHAIN_DOT branch of
    the reference's dot test (python/test/unit/language/test_core.py:3142-3144, `tl.dot(z.to(w.dtype), w)`).
    When the intermediate row fits one tile (N <= 256 and W's N2 <= 256) this is ONE launch and z never
    leaves the registers (`mi355_gemm_chain`); wider intermediates are two products with the rounding in
    between."""
    assert a.dtype == b.dtype == w.dtype, "Incompatible dtypes"
    assert a.shape[1] == b.shape[0] and b.shape[1] == w.shape[0], "Incompatible dimensions"
    in_dt = _abi_dtype(a)
    M, K = a.shape
    N, N2 = w.shape
    if in_dt in (_lib.F16, _lib.BF16) and N <= 256 and N2 <= 256 and M > 0 and K > 0:
        for i, t in enumerate((a, b, w)):
            _check_device(i, t)
        if out_dtype is None:
            out_dtype = a.dtype
        if activation not in ("", "leaky_relu"):
            raise KeyError(f"unknown ACTIVATION {activation!r}")
        c = torch.empty((M, N2), device=a.device, dtype=out_dtype)
        d_ptr, d_sm, d_sn, d_dt = 0, 0, 0, 0
        if add is not None:
            d = torch.broadcast_to(add, (M, N))
            d_ptr, d_sm, d_sn, d_dt = d.data_ptr(), d.stride(0), d.stride(1), _TORCH_TO_ABI[add.dtype]
        rc = _lib.load().mi355_gemm_chain(
            a.data_ptr(), b.data_ptr(), w.data_ptr(), c.data_ptr(), M, N, K, N2,
            a.stride(0), a.stride(1), b.stride(0), b.stride(1), w.stride(0), w.stride(1), c.stride(0), c.stride(1),
            in_dt, _TORCH_TO_ABI[out_dtype], None, None, d_ptr, d_sm, d_sn, d_dt,
            _lib.ACT_LEAKY_RELU if activation == "leaky_relu" else _lib.ACT_NONE, int(bool(softmax)), _stream())
        _lib.check(rc, "mi355_gemm_chain")
        return c
    z = matmul(a, b, activation, out_dtype=a.dtype, add=add, softmax=softmax)
    return matmul(z, w, out_dtype=out_dtype)


def matmul_like_input(a, b):
    """`matmul(a, b)` of the persistent-matmul tutorial (09:105-138): result dtype = input dtype
    (fp16 -> fp16, fp8e4nv -> fp8e4nv); A need not be contiguous there."""
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.dtype == b.dtype, "Incompatible dtypes"
    in_dt = _abi_dtype(a)
    _check_device(0, a)
    _check_device(1, b)
    M, K = a.shape
    K, N = b.shape
    c = torch.empty((M, N), device=a.device, dtype=a.dtype)
    stream = _stream()
    md = hooks.enter("mi355_gemm", stream, hooks.matmul_launch_metadata, ("mi355_gemm", M, N, K, _ELEM_BYTES[in_dt]))
    rc = _lib.load().mi355_gemm(
        a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K,
        a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
        in_dt, in_dt, None, None, _lib.ACT_NONE, stream)
    _lib.check(rc, "mi355_gemm")
    hooks.exit(md)
    return c


def matmul_persistent(a, b):
    """`matmul_persistent(a, b)` of the same tutorial (09:190-224): NUM_SMS programs walk the tiles.
    Here that is the library's default for large products with whole 256x256 tiles (one program per
    CU, each walking its tiles as one stream of K steps), so this is the same call as
    `matmul_like_input`; other shapes run one workgroup per tile.  Same `a @ b` in the input dtype."""
    return matmul_like_input(a, b)


def group_gemm_fn(group_A, group_B, *, num_programs: int = 0):
    """The reference's `group_gemm_fn(group_A, group_B)` (python/tutorials/08-grouped-gemm.py:143-187):
    `[A_i @ B_i for i]` in one launch.  Builds the same five device tables (matrix addresses,
    <M, N, K>, <lda, ldb, ldc>) and hands them to the grouped kernel; outputs have A's dtype.
    fp16 as in the reference, or bf16.  `num_programs` is the reference's NUM_SM (0 = two per CU)."""
    assert len(group_A) == len(group_B)
    group_size = len(group_A)
    if group_size == 0:
        return []
    device = group_A[0].device
    dt = _abi_dtype(group_A[0])
    assert dt in (_lib.F16, _lib.BF16), "grouped GEMM takes fp16 or bf16 matrices"
    A_addrs, B_addrs, C_addrs, g_sizes, g_lds, group_C = [], [], [], [], [], []
    for i in range(group_size):
        A, B = group_A[i], group_B[i]
        _check_device(2 * i, A)
        _check_device(2 * i + 1, B)
        assert A.shape[1] == B.shape[0]
        assert A.dtype == B.dtype == group_A[0].dtype, "all matrices of a group share one dtype"
        assert A.stride(1) == 1 and B.stride(1) == 1, "matrices must be row major"
        M, K = A.shape
        K, N = B.shape
        C = torch.empty((M, N), device=device, dtype=A.dtype)
        group_C.append(C)
        A_addrs.append(A.data_ptr())
        B_addrs.append(B.data_ptr())
        C_addrs.append(C.data_ptr())
        g_sizes += [M, N, K]
        g_lds += [A.stride(0), B.stride(0), C.stride(0)]
    # device tables, as in the reference (08:166-170)
    d_a_ptrs = torch.tensor(A_addrs, device=device, dtype=torch.int64)
    d_b_ptrs = torch.tensor(B_addrs, device=device, dtype=torch.int64)
    d_c_ptrs = torch.tensor(C_addrs, device=device, dtype=torch.int64)
    d_g_sizes = torch.tensor(g_sizes, dtype=torch.int32, device=device)
    d_g_lds = torch.tensor(g_lds, dtype=torch.int32, device=device)
    rc = _lib.load().mi355_grouped_gemm(d_a_ptrs.data_ptr(), d_b_ptrs.data_ptr(), d_c_ptrs.data_ptr(),
                                        d_g_sizes.data_ptr(), d_g_lds.data_ptr(), group_size, dt,
                                        int(num_programs), _stream())
    _lib.check(rc, "mi355_grouped_gemm")
    return group_C


def mx_matmul(a_packed, a_scale, b_packed, b_scale, fmt="mxfp4", out_dtype=torch.bfloat16):
    """Block-scaled matmul C[M,N] = A[M,K] . B[N,K]^T (OCP MX v1.0, 32-element blocks along K).

    mxfp4: a_packed [M, K/2] / b_packed [N, K/2] uint8 (e2m1, element 2i in the low nibble);
    mxfp8: [M, K] / [N, K] float8_e4m3fn or uint8 codes; scales [M, K/32] / [N, K/32] uint8
    e8m0.  No counterpart in the reference snapshot.
    """
    f = {"mxfp4": _lib.MXFP4, "mxfp8": _lib.MXFP8}[fmt]
    for i, t in enumerate((a_packed, a_scale, b_packed, b_scale)):
        _check_device(i, t)
        assert t.dim() == 2 and t.stride(1) == 1, "operands and scales must be row-major 2-D"
        assert t.element_size() == 1, "packed operands and scales are byte tensors"
    M, KB = a_packed.shape
    N = b_packed.shape[0]
    K = KB * 2 if f == _lib.MXFP4 else KB
    assert b_packed.shape[1] == KB, "Incompatible dimensions"
    assert K % 32 == 0, "K must be a multiple of the 32-element scale block"
    assert tuple(a_scale.shape) == (M, K // 32) and tuple(b_scale.shape) == (N, K // 32), "scale shape must be [rows, K/32]"
    c = torch.empty((M, N), device=a_packed.device, dtype=out_dtype)
    ext = _lib.ext()
    if ext is not None:
        ext.mx_gemm(a_packed, a_scale, b_packed, b_scale, c, f, K)
        return c
    rc = _lib.load().mi355_mx_gemm(
        a_packed.data_ptr(), a_scale.data_ptr(), b_packed.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
        M, N, K, f, _TORCH_TO_ABI[out_dtype],
        a_packed.stride(0), b_packed.stride(0), a_scale.stride(0), b_scale.stride(0), c.stride(0), _stream())
    _lib.check(rc, "mi355_mx_gemm")
    return c


def dequantize(codes: torch.Tensor, fmt: str) -> torch.Tensor:
    """Decode narrow-format codes on the GPU with the kernels' own decode routines.
    fmt: 'e4m3' | 'e5m2' | 'e8m0' (one value per byte) or 'e2m1' (two per byte, low nibble first)."""
    f = {"e4m3": _lib.DEQ_E4M3, "e5m2": _lib.DEQ_E5M2, "e2m1": _lib.DEQ_E2M1, "e8m0": _lib.DEQ_E8M0}[fmt]
    _check_device(0, codes)
    assert codes.is_contiguous() and codes.element_size() == 1
    n = codes.numel()
    shape = list(codes.shape)
    if f == _lib.DEQ_E2M1:
        shape[-1] *= 2
    out = torch.empty(shape, dtype=torch.float32, device=codes.device)
    if n:
        _lib.check(_lib.load().mi355_dequant(codes.data_ptr(), out.data_ptr(), n, f, _stream()), "mi355_dequant")
    return out


class _attention(torch.autograd.Function):
    """Autograd function with the reference's forward/backward split (06:438-517)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale):
        HEAD_DIM_Q, HEAD_DIM_K = q.shape[-1], k.shape[-1]
        HEAD_DIM_V = v.shape[-1]
        assert HEAD_DIM_Q == HEAD_DIM_K and HEAD_DIM_K == HEAD_DIM_V
        assert HEAD_DIM_K in {16, 32, 64, 128, 256}
        for i, t in enumerate((q, k, v)):
            _check_device(i, t)
        assert q.dtype == k.dtype == v.dtype, "q, k, v must share a dtype"
        dt = _abi_dtype(q)
        if dt in (_lib.F8E4M3, _lib.F8E5M2):
            # the reference passes V transposed in memory for fp8 (06:609-614) and has no fp8 backward
            assert v.stride(2) == 1, "fp8 attention takes v transposed in memory: v.permute(0,1,3,2).contiguous().permute(0,1,3,2)"
            assert not (q.requires_grad or k.requires_grad or v.requires_grad), "fp8 attention is forward only"
        o = torch.empty_like(q)
        Z, H, N_CTX = q.shape[0], q.shape[1], q.shape[2]
        M = torch.empty((Z, H, N_CTX), device=q.device, dtype=torch.float32)
        I4 = _lib.I64x4
        stream = _stream()
        md = hooks.enter("mi355_attn_fwd", stream, hooks.attention_launch_metadata,
                         ("mi355_attn_fwd", Z, H, N_CTX, HEAD_DIM_K, causal, _ELEM_BYTES[dt]))
        ext = _lib.ext()
        if ext is not None:
            ext.attn_fwd(q, k, v, o, M, float(sm_scale), bool(causal))
        else:
            rc = _lib.load().mi355_attn_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), M.data_ptr(),
                Z, H, N_CTX, HEAD_DIM_K,
                I4(*q.stride()), I4(*k.stride()), I4(*v.stride()), I4(*o.stride()),
                float(sm_scale), int(bool(causal)), dt, stream)
            _lib.check(rc, "mi355_attn_fwd")
        hooks.exit(md)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.sm_scale = sm_scale
        ctx.HEAD_DIM = HEAD_DIM_K
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, M = ctx.saved_tensors
        assert do.is_contiguous()
        assert q.stride() == k.stride() == v.stride() == o.stride() == do.stride()
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        BATCH, N_HEAD, N_CTX = q.shape[:3]
        PRE_BLOCK = 128
        assert N_CTX % PRE_BLOCK == 0
        delta = torch.empty_like(M)
        dt = _abi_dtype(q)
        ext = _lib.ext()
        if ext is not None:
            ext.attn_bwd(q, k, v, o, do, M, delta, dq, dk, dv, float(ctx.sm_scale), bool(ctx.causal))
            return dq, dk, dv, None, None
        I4 = _lib.I64x4
        lib = _lib.load()
        rc = lib.mi355_attn_bwd_preprocess(
            o.data_ptr(), do.data_ptr(), delta.data_ptr(), BATCH, N_HEAD, N_CTX, ctx.HEAD_DIM,
            I4(*o.stride()), dt, _stream())
        _lib.check(rc, "mi355_attn_bwd_preprocess")
        rc = lib.mi355_attn_bwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), M.data_ptr(), delta.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), BATCH, N_HEAD, N_CTX, ctx.HEAD_DIM,
            I4(*q.stride()), float(ctx.sm_scale), int(bool(ctx.causal)), dt, _stream())
        _lib.check(rc, "mi355_attn_bwd")
        return dq, dk, dv, None, None


def attention(q, k, v, causal, sm_scale):
    """`attention(q, k, v, causal, sm_scale)` of the reference (06:520, `_attention.apply`).

    Head dims 64, 128 and 256 have kernels of their own, forward and backward.  The reference also admits 16
    and 32 (06:447): those run the 64-column kernels in a form that pads with zeros on the fly - the rows are
    loaded as they are (32 or 64 bytes), the missing columns never exist in memory, and only the first
    HEAD_DIM columns of every output and gradient are stored - so no padded copies are made."""
    return _attention.apply(q, k, v, causal, sm_scale)


def default_sm_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
