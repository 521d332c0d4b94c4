"""Tensor-level wrappers over the C ABI: shape checks, output allocation, one call each."""
import torch

from . import _lib as L

SWIGLU_EPILOGUE_MIN_M = 512      # rows from which the gate/up contraction runs tiled and can carry the swiglu in its epilogue
GEMV_MAX_M = 8      # rows handled by the fused norm+quant+GEMV launch (every workgroup redoes the row's prologue,
                    # which stops paying off around 8 rows); above: quantise once per row, then the matrix cores

_workspaces = {}


def _workspace(device, nbytes, tag):
    key = (device, tag)
    w = _workspaces.get(key)
    if w is None or w.numel() < nbytes:
        w = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _workspaces[key] = w
    return w


def _as_2d(x):
    return x.reshape(-1, x.shape[-1]).contiguous()


# ------------------------------------------------------------------------------ weights
class PackedWeight:
    """2-bit packed ternary codes of one or more [N_i, K] matrices stacked along N."""

    def __init__(self, packed, wdeq, n, k, seg_rows):
        self.packed, self.wdeq, self.n, self.k, self.seg_rows = packed, wdeq, n, k, seg_rows

    @property
    def nbytes(self):
        return self.packed.numel()


def ternarize_pack(weight):
    """weight [N, K] (fp32/bf16/fp16, CUDA) -> PackedWeight."""
    L.require_gpu(weight)
    lib = L.load()
    w = weight.detach().contiguous()
    n, k = w.shape
    packed = torch.empty(lib.mmf_packed_bytes(n, k), dtype=torch.uint8, device=w.device)
    wdeq = torch.empty(1, dtype=torch.float32, device=w.device)
    ws = _workspace(w.device, lib.mmf_ternarize_workspace_bytes(), "tern")
    with torch.cuda.device(w.device):
        L.check(lib.mmf_ternarize_pack(w.data_ptr(), L.dtype_id(w.dtype), n, k, packed.data_ptr(), wdeq.data_ptr(),
                                       ws.data_ptr(), L.stream()), "mmf_ternarize_pack")
    return PackedWeight(packed, wdeq, n, k, -(-n // 32) * 32)


def stack_packed(parts):
    """Concatenate PackedWeights with equal K and row counts that are multiples of 32."""
    k = parts[0].k
    assert all(p.k == k for p in parts) and all(p.n == parts[0].n and p.n % 32 == 0 for p in parts)
    return PackedWeight(torch.cat([p.packed for p in parts]), torch.cat([p.wdeq for p in parts]),
                        sum(p.n for p in parts), k, parts[0].n)


def unpack_ternary(pw):
    lib = L.load()
    codes = torch.empty(pw.n, pw.k, dtype=torch.int8, device=pw.packed.device)
    with torch.cuda.device(codes.device):
        L.check(lib.mmf_unpack_ternary(pw.packed.data_ptr(), pw.n, pw.k, codes.data_ptr(), L.stream()), "mmf_unpack_ternary")
    return codes


# ------------------------------------------------------------------------------ norms
def _norm_common(x, residual, weight, prenorm, residual_in_fp32, keep_strided=False):
    dev = L.require_gpu(x, residual, weight)
    shp = x.shape
    x2 = x if keep_strided else _as_2d(x)
    r2 = None
    if residual is not None:
        if residual.numel() != x.numel():
            raise ValueError(f"residual shape {tuple(residual.shape)} != x shape {tuple(shp)}")
        r2 = _as_2d(residual)
    if r2 is not None and r2.shape != (x2.shape[0], x2.shape[1]):
        raise ValueError("residual does not match x")
    res_dtype = r2.dtype if r2 is not None else (torch.float32 if residual_in_fp32 else x2.dtype)
    need_res_out = r2 is not None or res_dtype != x2.dtype
    # the summed residual stream is only materialised when the caller asks for it back (prenorm)
    res_out = torch.empty(tuple(x2.shape), dtype=res_dtype, device=dev) if (need_res_out and prenorm) else None
    w = weight.detach().contiguous() if weight is not None else None
    return dev, shp, x2, r2, res_dtype, res_out, w


def rmsnorm(x, weight, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False):
    """RMSNorm with optional fused residual add; returns y or (y, residual_out) if prenorm."""
    lib = L.load()
    dev, shp, x2, r2, res_dtype, res_out, w = _norm_common(x, residual, weight, prenorm, residual_in_fp32)
    y = torch.empty_like(x2)
    m, k = x2.shape
    with torch.cuda.device(dev):
        L.check(lib.mmf_rmsnorm(x2.data_ptr(), L.ptr(r2), L.ptr(w), y.data_ptr(), L.ptr(res_out), m, k, eps,
                                L.dtype_id(x2.dtype), L.dtype_id(res_dtype), L.dtype_id(w.dtype) if w is not None else 0,
                                L.stream()), "mmf_rmsnorm")
    y = y.reshape(shp)
    if not prenorm:
        return y
    return y, (res_out.reshape(shp) if res_out is not None else x)


def rmsnorm_swishgate(x, o, weight, residual=None, eps=1e-6, prenorm=False, residual_in_fp32=False):
    """y = RMSNorm(x [+ residual]) * weight * o * sigmoid(o)."""
    lib = L.load()
    L.require_gpu(o)
    if o.shape != x.shape or o.dtype != x.dtype:
        raise ValueError("gate tensor must match x in shape and dtype")
    k = x.shape[-1]
    x_view, _, ldx = _rows_ld(x, k)      # x may be a column slice of a wider matrix
    dev, shp, x2, r2, res_dtype, res_out, w = _norm_common(x_view if ldx != k else x, residual, weight, prenorm,
                                                           residual_in_fp32, keep_strided=ldx != k)
    shp = x.shape
    o2 = _as_2d(o)
    m = x2.shape[0]
    y = torch.empty(m, k, dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_rmsnorm_swishgate(x2.data_ptr(), ldx, o2.data_ptr(), L.ptr(r2), L.ptr(w), y.data_ptr(), L.ptr(res_out),
                                          m, k, eps, L.dtype_id(x2.dtype), L.dtype_id(res_dtype),
                                          L.dtype_id(w.dtype) if w is not None else 0, L.stream()), "mmf_rmsnorm_swishgate")
    y = y.reshape(shp)
    if not prenorm:
        return y
    return y, (res_out.reshape(shp) if res_out is not None else x)


def swiglu(x, y):
    """(x * y) / (1 + exp(-x)); x and y may be last-dim slices of one wider tensor."""
    lib = L.load()
    dev = L.require_gpu(x, y)
    if x.shape != y.shape or x.dtype != y.dtype:
        raise ValueError("swiglu operands must match in shape and dtype")
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)

    def view2d(t):
        # keep a column slice of a contiguous wider matrix as (ptr, ld) instead of copying it
        if t.dim() >= 1 and t.stride(-1) == 1 and rows > 0:
            t2 = t.reshape(rows, cols) if t.is_contiguous() else None
            if t2 is None:
                try:
                    t2 = t.view(rows, cols)
                except RuntimeError:
                    t2 = None
            if t2 is not None and t2.stride(1) == 1:
                return t2, (t2.stride(0) if rows > 1 else cols)
        t2 = t.reshape(rows, cols).contiguous()
        return t2, cols

    x2, ldx = view2d(x)
    y2, ldy = view2d(y)
    out = torch.empty(x.shape, dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_swiglu(x2.data_ptr(), ldx, y2.data_ptr(), ldy, out.data_ptr(), rows, cols, L.dtype_id(x.dtype),
                               L.stream()), "mmf_swiglu")
    return out


def rmsnorm_quant(x, weight, residual=None, eps=1e-8, tiled=False, prenorm=False, residual_in_fp32=False,
                  norm_bias=None, is_rms_norm=True):
    """RMSNorm + per-row absmax int8 codes.  Returns (q uint8-storage int8 tensor, deq, qsum[, residual_out]).

    q is [M, Kp] (row-major) or the flat tiled buffer when tiled=True; Kp = ceil128(K).
    is_rms_norm=False: LayerNorm (row mean subtracted first) with an optional norm_bias in the weight's dtype.
    """
    lib = L.load()
    dev, shp, x2, r2, res_dtype, res_out, w = _norm_common(x, residual, weight, prenorm, residual_in_fp32)
    if not is_rms_norm:
        return _layernorm_quant(lib, dev, shp, x, x2, r2, res_dtype, res_out, w, norm_bias, eps, tiled, prenorm)
    if norm_bias is not None:
        raise ValueError("norm_bias needs is_rms_norm=False (the RMSNorm of the BitLinear path has no bias)")
    m, k = x2.shape
    if (tiled and r2 is None and res_out is None and m > 256 and k % 4 == 0 and k <= 8192
            and (w is None or w.dtype in (x2.dtype, torch.float32))):
        # many rows: the form that puts several rows in a workgroup (one wave per 2048 elements of a row)
        q = torch.empty(lib.mmf_codes_bytes(m, k, 1), dtype=torch.int8, device=dev)
        deq = torch.empty(m, dtype=torch.float32, device=dev)
        qsum = torch.empty(m, dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            L.check(lib.mmf_rmsnorm_quant_fused(0, x2.data_ptr(), x2.stride(0), None, 0, None, 0, None, None, 0.0, L.ptr(w), eps,
                                                None, None, q.data_ptr(), deq.data_ptr(), qsum.data_ptr(), m, k,
                                                L.dtype_id(x2.dtype), L.dtype_id(w.dtype) if w is not None else 0, L.stream()),
                    "mmf_rmsnorm_quant_fused")
        return (q, deq, qsum, x) if prenorm else (q, deq, qsum)
    kp = -(-k // 128) * 128
    nbytes = lib.mmf_codes_bytes(m, k, 1 if tiled else 0)
    q = torch.empty(nbytes, dtype=torch.int8, device=dev)
    deq = torch.empty(m, dtype=torch.float32, device=dev)
    qsum = torch.empty(m, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_rmsnorm_quant(x2.data_ptr(), L.ptr(r2), L.ptr(w), q.data_ptr(), deq.data_ptr(), qsum.data_ptr(),
                                      L.ptr(res_out), m, k, eps, L.dtype_id(x2.dtype), L.dtype_id(res_dtype),
                                      L.dtype_id(w.dtype) if w is not None else 0, 1 if tiled else 0, L.stream()),
                "mmf_rmsnorm_quant")
    if not tiled:
        q = q.view(m, kp)
    if prenorm:
        return q, deq, qsum, (res_out.reshape(shp) if res_out is not None else x)
    return q, deq, qsum


def _layernorm_quant(lib, dev, shp, x, x2, r2, res_dtype, res_out, w, bias, eps, tiled, prenorm):
    m, k = x2.shape
    if bias is not None:
        if w is None:
            raise ValueError("a norm bias needs a norm weight (they share a dtype)")
        L.require_gpu(bias)
        bias = bias.detach().to(w.dtype).contiguous()
        if bias.shape != (k,):
            raise ValueError(f"norm bias has shape {tuple(bias.shape)}, expected ({k},)")
    q = torch.empty(lib.mmf_codes_bytes(m, k, 1 if tiled else 0), dtype=torch.int8, device=dev)
    deq = torch.empty(m, dtype=torch.float32, device=dev)
    qsum = torch.empty(m, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_layernorm_quant(x2.data_ptr(), L.ptr(r2), L.ptr(w), L.ptr(bias), q.data_ptr(), deq.data_ptr(),
                                        qsum.data_ptr(), L.ptr(res_out), m, k, eps, L.dtype_id(x2.dtype),
                                        L.dtype_id(res_dtype), L.dtype_id(w.dtype) if w is not None else 0,
                                        1 if tiled else 0, L.stream()), "mmf_layernorm_quant")
    if not tiled:
        q = q.view(m, -(-k // 128) * 128)
    if prenorm:
        return q, deq, qsum, (res_out.reshape(shp) if res_out is not None else x)
    return q, deq, qsum


def codes_tiled_to_rowmajor(q_tiled, m, k):
    """Undo the matrix-core tiling: flat [ceil32(M)/32][Kp/16][32][16] -> [M, K]."""
    kp = -(-k // 128) * 128
    mp = -(-m // 32) * 32
    t = q_tiled.view(mp // 32, kp // 16, 32, 16).permute(0, 2, 1, 3).reshape(mp, kp)
    return t[:m, :k]


# ------------------------------------------------------------------------------ BitLinear
def bitlinear_mfma(q_tiled, deq, qsum, pw, m, out_dtype, bias=None, config=-1, out=None, addend=None):
    lib = L.load()
    dev = L.require_gpu(q_tiled, deq, qsum, pw.packed, bias)
    if out is None:
        out = torch.empty(m, pw.n, dtype=out_dtype, device=dev)
    ldo = out.stride(0) if m > 1 else max(out.shape[-1], pw.n)
    if bias is not None:
        bias = bias.detach().to(out_dtype).contiguous()
    if addend is not None:
        addend = addend.reshape(m, pw.n)
        if addend.dtype != out_dtype or not addend.is_contiguous() or ldo != pw.n:
            raise ValueError("addend must be a contiguous [M, N] tensor of the output dtype")
    with torch.cuda.device(dev):
        L.check(lib.mmf_bitlinear_mfma(q_tiled.data_ptr(), deq.data_ptr(), qsum.data_ptr(), pw.packed.data_ptr(),
                                       pw.wdeq.data_ptr(), pw.seg_rows, L.ptr(bias), L.ptr(addend), out.data_ptr(), ldo, m, pw.k, pw.n,
                                       L.dtype_id(out_dtype), config, L.stream()), "mmf_bitlinear_mfma")
    return out


def bitlinear_mfma_swiglu(q_tiled, deq, qsum, pw, m, out_dtype):
    """The tiled matrix-core contraction on the stacked [gate; up] weight with swiglu in its epilogue -> [m, N/2]."""
    lib = L.load()
    dev = L.require_gpu(q_tiled, deq, qsum, pw.packed)
    inter = pw.n // 2
    out = torch.empty(m, inter, dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_bitlinear_mfma_swiglu(q_tiled.data_ptr(), deq.data_ptr(), qsum.data_ptr(), pw.packed.data_ptr(),
                                              pw.wdeq.data_ptr(), pw.seg_rows, out.data_ptr(), inter, m, pw.k, pw.n,
                                              L.dtype_id(out_dtype), L.stream()), "mmf_bitlinear_mfma_swiglu")
    return out


def swiglu_epilogue_fits(m, pw, dtype):
    """Whether bitlinear_mfma_swiglu serves this problem: enough rows for the tiled kernel, whole 32-channel blocks,
    16-byte rows of the result."""
    inter = pw.n // 2
    return m >= SWIGLU_EPILOGUE_MIN_M and pw.n % 64 == 0 and inter % (4 if dtype == torch.float32 else 8) == 0


def bitlinear_gemv(x2, norm_weight, pw, eps, bias=None, addend=None):
    lib = L.load()
    dev = L.require_gpu(x2, norm_weight, pw.packed, bias)
    m, k = x2.shape
    out = torch.empty(m, pw.n, dtype=x2.dtype, device=dev)
    nw = norm_weight.detach().contiguous() if norm_weight is not None else None
    if bias is not None:
        bias = bias.detach().to(x2.dtype).contiguous()
    if addend is not None:
        addend = addend.reshape(m, pw.n)
        if addend.dtype != x2.dtype or not addend.is_contiguous():
            raise ValueError("addend must be a contiguous [M, N] tensor of the input dtype")
    with torch.cuda.device(dev):
        L.check(lib.mmf_bitlinear_gemv(x2.data_ptr(), L.ptr(nw), pw.packed.data_ptr(), pw.wdeq.data_ptr(), pw.seg_rows,
                                       L.ptr(bias), L.ptr(addend), out.data_ptr(), m, k, pw.n, eps, L.dtype_id(x2.dtype),
                                       L.dtype_id(nw.dtype) if nw is not None else 0, L.stream()), "mmf_bitlinear_gemv")
    return out


# prologue kinds -> (GEMV prologue id, fused-quantiser prologue id), include/mmf.h
_PROLOGUES = {"norm": (1, 1), "resnorm": (2, 2), "gatednorm": (3, 5), "swiglu": (4, 4)}


def _bitlinear_prologue(x, norm_weight, pw, bias, eps, addend, prologue, epilogue=None):
    """BitLinear with the op in front of it folded into the same launch (M <= GEMV_MAX_M) or into the quantiser
    (larger M).  prologue: ("norm", w1, eps1) | ("resnorm", residual, w1, eps1) | ("gatednorm", gate, w1, eps1)
    | ("swiglu", up).  x and the second operand may be column slices of a wider tensor.
    Returns out, or (out, summed_residual) for "resnorm"."""
    lib = L.load()
    kind = prologue[0]
    gid, qid = _PROLOGUES[kind]
    aux = prologue[1] if kind != "norm" else None
    w1 = prologue[-2] if kind != "swiglu" else None
    eps1 = float(prologue[-1]) if kind != "swiglu" else 0.0
    dev = L.require_gpu(x, aux, norm_weight, w1, pw.packed, bias)
    shp = x.shape
    k = shp[-1]
    if k != pw.k:
        raise ValueError(f"input features {k} != weight in_features {pw.k}")

    def rows(t):                                                # [M, K] view; column slices keep their row stride
        t2 = t.reshape(-1, k)
        return t2 if t2.stride(-1) == 1 else t2.contiguous()

    x2 = rows(x)
    a2 = rows(aux) if aux is not None else None
    m = x2.shape[0]
    if a2 is not None and (a2.shape != x2.shape or a2.dtype != x2.dtype):
        raise ValueError("the prologue operand must match x in shape and dtype")
    nw = norm_weight.detach().contiguous() if norm_weight is not None else None
    w1c = w1.detach().contiguous() if w1 is not None else None
    wdt = nw.dtype if nw is not None else (w1c.dtype if w1c is not None else torch.float32)
    if w1c is not None and nw is not None and w1c.dtype != nw.dtype:
        raise ValueError("the two norm weights must share a dtype")
    res_out = torch.empty(m, k, dtype=x2.dtype, device=dev) if kind == "resnorm" else None
    if epilogue is not None:
        _check_swiglu_epilogue(epilogue, m, pw, x2.dtype, bias, addend)
    out = torch.empty(m, pw.n, dtype=x2.dtype, device=dev) if epilogue is None else None
    if bias is not None:
        bias = bias.detach().to(x2.dtype).contiguous()
    if addend is not None:
        addend = addend.reshape(m, pw.n)
        if addend.dtype != x2.dtype or not addend.is_contiguous():
            raise ValueError("addend must be a contiguous [M, N] tensor of the input dtype")
    ldx = x2.stride(0) if m > 1 else k
    lda = (a2.stride(0) if m > 1 else k) if a2 is not None else 0
    with torch.cuda.device(dev):
        if m <= GEMV_MAX_M and k <= lib.mmf_bitlinear_gemv_max_k():
            L.check(lib.mmf_bitlinear_gemv_fused(gid, 0, x2.data_ptr(), ldx, L.ptr(a2), lda, L.ptr(res_out), L.ptr(w1c), eps1,
                                                 L.ptr(nw), eps, pw.packed.data_ptr(), pw.wdeq.data_ptr(), pw.seg_rows,
                                                 L.ptr(bias), L.ptr(addend), out.data_ptr(), None, None, None, m, k, pw.n,
                                                 L.dtype_id(x2.dtype), L.dtype_id(wdt), L.stream()), "mmf_bitlinear_gemv_fused")
        else:
            q = torch.empty(lib.mmf_codes_bytes(m, k, 1), dtype=torch.int8, device=dev)
            deq = torch.empty(m, dtype=torch.float32, device=dev)
            qsum = torch.empty(m, dtype=torch.int32, device=dev)
            L.check(lib.mmf_rmsnorm_quant_fused(qid, x2.data_ptr(), ldx, L.ptr(a2), lda, None, 0, L.ptr(res_out), L.ptr(w1c), eps1,
                                                L.ptr(nw), eps, None, None, q.data_ptr(), deq.data_ptr(), qsum.data_ptr(), m, k,
                                                L.dtype_id(x2.dtype), L.dtype_id(wdt), L.stream()), "mmf_rmsnorm_quant_fused")
            if epilogue is None:
                bitlinear_mfma(q, deq, qsum, pw, m, x2.dtype, bias, out=out, addend=addend)
            else:
                out = bitlinear_mfma_swiglu(q, deq, qsum, pw, m, x2.dtype)
    out = out.reshape(*shp[:-1], out.shape[-1])
    return (out, res_out.reshape(shp)) if kind == "resnorm" else out


def _check_swiglu_epilogue(epilogue, m, pw, dtype, bias, addend):
    if epilogue != "swiglu":
        raise ValueError("epilogue must be None or 'swiglu'")
    if bias is not None or addend is not None or not swiglu_epilogue_fits(m, pw, dtype):
        raise ValueError("the swiglu epilogue takes no bias or addend and needs swiglu_epilogue_fits(m, weight, dtype)")


def bitlinear(x, norm_weight, pw, bias=None, eps=1e-8, residual=None, prenorm=False, residual_in_fp32=False,
              path=None, addend=None, prologue=None, epilogue=None, norm_bias=None, is_rms_norm=True):
    """Fused BitLinear forward on x [..., K] -> [..., N] (x.dtype).

    is_rms_norm=False (with an optional norm_bias): the LayerNorm form; it always takes the quantiser + contraction
    pair of launches.

    path: None (by M), "gemv" or "mfma".  With a residual (or prenorm) the two-launch path is used.
    prologue: see _bitlinear_prologue (the elementwise op that produces this BitLinear's input, fused).
    epilogue: "swiglu" on a stacked [gate; up] weight returns swiglu(gate, up) [..., N/2] from the contraction's own
    epilogue (large M only: swiglu_epilogue_fits).
    """
    if prologue is not None:
        if residual is not None or prenorm or path is not None or not is_rms_norm:
            raise ValueError("prologue= excludes residual=, prenorm=, path= and the LayerNorm form")
        return _bitlinear_prologue(x, norm_weight, pw, bias, eps, addend, prologue, epilogue)
    lib = L.load()
    L.require_gpu(x)
    shp = x.shape
    k = shp[-1]
    if k != pw.k:
        raise ValueError(f"input features {k} != weight in_features {pw.k}")
    x2 = _as_2d(x)
    m = x2.shape[0]
    plain = residual is None and not prenorm and is_rms_norm
    if not is_rms_norm and path == "gemv":
        raise ValueError("the fused GEMV launch has the RMSNorm form only")
    if path is None:
        path = "gemv" if (plain and m <= GEMV_MAX_M and k <= lib.mmf_bitlinear_gemv_max_k()) else "mfma"
    if path == "gemv":
        if not plain:
            raise ValueError("the fused GEMV launch takes no residual")
        out = bitlinear_gemv(x2, norm_weight, pw, eps, bias, addend)
        return out.reshape(*shp[:-1], pw.n)
    res = rmsnorm_quant(x, norm_weight, residual=residual, eps=eps, tiled=True, prenorm=prenorm,
                        residual_in_fp32=residual_in_fp32, norm_bias=norm_bias, is_rms_norm=is_rms_norm)
    q, deq, qsum = res[:3]
    if epilogue is not None:
        _check_swiglu_epilogue(epilogue, m, pw, x.dtype, bias, addend)
        out = bitlinear_mfma_swiglu(q, deq, qsum, pw, m, x.dtype).reshape(*shp[:-1], pw.n // 2)
    else:
        out = bitlinear_mfma(q, deq, qsum, pw, m, x.dtype, bias, addend=addend).reshape(*shp[:-1], pw.n)
    return (out, res[3]) if prenorm else out


# ------------------------------------------------------------------------------ HGRN
def _state32(h0, bh, d, dev):
    if h0 is None:
        return None
    return h0.detach().reshape(bh, d).to(device=dev, dtype=torch.float32).contiguous()


def hgrn_recurrent(x, g, initial_state=None, output_final_state=False):
    """x, g [B, H, T, D]; g is the decay itself.  Returns (o, final_state fp32 [B, H, D] or None)."""
    lib = L.load()
    dev = L.require_gpu(x, g, initial_state)
    if x.shape != g.shape or x.dtype != g.dtype or x.dim() != 4:
        raise ValueError("x and g must be [B, H, T, D] tensors of one dtype")
    b, h, t, d = x.shape
    xc, gc = x.contiguous(), g.contiguous()
    o = torch.empty_like(xc)
    h0 = _state32(initial_state, b * h, d, dev)
    ht = torch.empty(b, h, d, dtype=torch.float32, device=dev) if output_final_state else None
    with torch.cuda.device(dev):
        L.check(lib.mmf_hgrn_recurrent(xc.data_ptr(), gc.data_ptr(), L.ptr(h0), o.data_ptr(), L.ptr(ht), b * h, t, d,
                                       L.dtype_id(x.dtype), L.stream()), "mmf_hgrn_recurrent")
    return o, ht


def hgrn_chunk(x, g, initial_state=None, output_final_state=False, chunk_size=64):
    """x, g [B, H, T, D]; g is the LOG decay.  Returns (o, final_state fp32 or None)."""
    lib = L.load()
    dev = L.require_gpu(x, g, initial_state)
    if x.shape != g.shape or x.dtype != g.dtype or x.dim() != 4:
        raise ValueError("x and g must be [B, H, T, D] tensors of one dtype")
    b, h, t, d = x.shape
    xc, gc = x.contiguous(), g.contiguous()
    o = torch.empty_like(xc)
    h0 = _state32(initial_state, b * h, d, dev)
    ht = torch.empty(b, h, d, dtype=torch.float32, device=dev) if output_final_state else None
    if not 1 <= chunk_size <= 64:
        raise ValueError("chunk_size must lie in [1, 64]")
    nws = lib.mmf_hgrn_chunk_workspace_bytes(b * h, t, d, chunk_size)
    ws = torch.empty(nws // 4, dtype=torch.float32, device=dev) if nws else None    # per-segment carries (few KB)
    with torch.cuda.device(dev):
        L.check(lib.mmf_hgrn_chunk(xc.data_ptr(), gc.data_ptr(), L.ptr(h0), o.data_ptr(), L.ptr(ht), b * h, t, d,
                                   chunk_size, L.dtype_id(x.dtype), L.ptr(ws), L.stream()), "mmf_hgrn_chunk")
    return o, ht


def _rows_ld(t, d):
    """[..., D] tensor, possibly a column slice of a wider contiguous matrix -> (tensor, rows, ld)."""
    rows = t.numel() // d
    if t.stride(-1) == 1:
        try:
            t2 = t.view(rows, d) if not t.is_contiguous() else t.reshape(rows, d)
            return t2, rows, (t2.stride(0) if rows > 1 else d)
        except RuntimeError:
            pass
    t2 = t.reshape(rows, d).contiguous()
    return t2, rows, d


def _mask_rows(mask, rows, dev):
    if mask is None:
        return None
    m = (mask.reshape(-1) != 0).to(device=dev, dtype=torch.uint8).contiguous()
    if m.numel() != rows:
        raise ValueError("attention mask does not match the token count")
    return m


def hgrn_gate(i, f, lower_bound=None, attention_mask=None):
    """Fused sigmoid / lower bound / swiglu / mask.  i, f [..., D] -> (x, g) contiguous [..., D]."""
    lib = L.load()
    dev = L.require_gpu(i, f, lower_bound)
    d = i.shape[-1]
    i2, rows, ldi = _rows_ld(i, d)
    f2, _, ldf = _rows_ld(f, d)
    lb = lower_bound.detach().to(torch.float32).contiguous() if lower_bound is not None else None
    mk = _mask_rows(attention_mask, rows, dev)
    xo = torch.empty(i.shape, dtype=i.dtype, device=dev)
    go = torch.empty(i.shape, dtype=i.dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_hgrn_gate(i2.data_ptr(), ldi, f2.data_ptr(), ldf, L.ptr(lb), L.ptr(mk), xo.data_ptr(),
                                  go.data_ptr(), rows, d, L.dtype_id(i.dtype), L.stream()), "mmf_hgrn_gate")
    return xo, go


def hgrn_step(i, f, state, lower_bound=None, attention_mask=None):
    """One decode step: gate math + h = g*h + x.  state fp32 [rows, D] is updated in place; returns o."""
    lib = L.load()
    dev = L.require_gpu(i, f, state, lower_bound)
    d = i.shape[-1]
    i2, rows, ldi = _rows_ld(i, d)
    f2, _, ldf = _rows_ld(f, d)
    if state.dtype != torch.float32 or not state.is_contiguous() or state.numel() != rows * d:
        raise ValueError("state must be a contiguous fp32 tensor of rows*D elements")
    lb = lower_bound.detach().to(torch.float32).contiguous() if lower_bound is not None else None
    mk = _mask_rows(attention_mask, rows, dev)
    o = torch.empty(i.shape, dtype=i.dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_hgrn_step(i2.data_ptr(), ldi, f2.data_ptr(), ldf, L.ptr(lb), L.ptr(mk), state.data_ptr(),
                                  o.data_ptr(), rows, d, L.dtype_id(i.dtype), L.stream()), "mmf_hgrn_step")
    return o


# ------------------------------------------------------------------------------ decode ends
def embedding(table, ids):
    """table [V, H], ids int64 [...] -> [..., H]."""
    lib = L.load()
    dev = L.require_gpu(table, ids)
    idc = ids.reshape(-1).to(torch.int64).contiguous()
    tb = table.detach().contiguous()
    out = torch.empty(idc.numel(), tb.shape[1], dtype=tb.dtype, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_embedding(tb.data_ptr(), idc.data_ptr(), out.data_ptr(), idc.numel(), tb.shape[1], tb.shape[0],
                                  L.dtype_id(tb.dtype), L.stream()), "mmf_embedding")
    return out.reshape(*ids.shape, tb.shape[1])


def argmax(logits):
    """Lowest index of the maximum over the last dim; logits [..., V] -> int64 [...]."""
    lib = L.load()
    dev = L.require_gpu(logits)
    v = logits.shape[-1]
    l2 = _as_2d(logits)
    out = torch.empty(l2.shape[0], dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_argmax(l2.data_ptr(), v, l2.shape[0], v, out.data_ptr(), L.dtype_id(l2.dtype), L.stream()),
                "mmf_argmax")
    return out.reshape(logits.shape[:-1])


def sample_top_p(logits, top_p, temperature, u, out=None, top_k=0):
    """One top-k / top-p (nucleus) draw per row; logits [..., V], u fp32 [...] uniform in [0, 1) -> int64 [...].
    top_k > 0 keeps the top_k most probable tokens before the nucleus is taken (0: no limit).

    What transformers' sampling path does per token for the reference's generate.py:11 (temperature, softmax,
    sort, cumulative sum, nucleus mask, multinomial), as one launch: integer probability masses decide the nucleus
    and the draw is the inverse CDF of u over the kept tokens in index order (include/mmf.h gives the arithmetic).
    The caller owns the random stream: u = torch.rand(..., generator=g)."""
    lib = L.load()
    dev = L.require_gpu(logits)
    v = logits.shape[-1]
    l2 = _as_2d(logits)
    rows = l2.shape[0]
    if not (isinstance(u, torch.Tensor) and u.dtype == torch.float32 and u.device == dev and u.numel() == rows):
        raise L.MMFError("sample_top_p: u must be an fp32 tensor on the logits' device with one number per row")
    if not u.is_contiguous():
        u = u.contiguous()
    if out is None:
        out = torch.empty(rows, dtype=torch.int64, device=dev)
    elif not (out.dtype == torch.int64 and out.device == dev and out.numel() == rows and out.is_contiguous()):
        raise L.MMFError("sample_top_p: out must be a contiguous int64 tensor with one element per row")
    with torch.cuda.device(dev):
        L.check(lib.mmf_sample_top_p(l2.data_ptr(), l2.stride(0), rows, v, float(temperature), float(top_p), int(top_k),
                                     u.data_ptr(), out.data_ptr(), L.dtype_id(l2.dtype), L.stream()), "mmf_sample_top_p")
    return out.reshape(logits.shape[:-1])


def sample_top_p_max_vocab():
    """Widest row sample_top_p accepts."""
    return int(L.load().mmf_sample_top_p_max_vocab())


def cross_entropy(logits, labels, ignore_index=-100):
    """Mean next-token cross entropy as nn.CrossEntropyLoss()(logits.view(-1, V), labels.view(-1)) gives it, computed
    in fp32 from logits of any supported dtype (forward only); labels int64, already shifted by the caller.
    Returns a 0-dim fp32 tensor (NaN when every label is ignored, as torch returns)."""
    lib = L.load()
    dev = L.require_gpu(logits, labels)
    v = logits.shape[-1]
    l2 = _as_2d(logits)
    lab = labels.reshape(-1).to(torch.int64).contiguous()
    if lab.numel() != l2.shape[0]:
        raise ValueError("one label per row of logits")
    rows = torch.empty(l2.shape[0], dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_cross_entropy_fwd(l2.data_ptr(), l2.stride(0), lab.data_ptr(), int(ignore_index), rows.data_ptr(),
                                          l2.shape[0], v, L.dtype_id(l2.dtype), L.stream()), "mmf_cross_entropy_fwd")
    counted = ((lab != ignore_index) & (lab >= 0) & (lab < v)).sum()
    return rows.sum() / counted


# ------------------------------------------------------------------------------ ShortConvolution
def _conv_args(x, weight, bias):
    dev = L.require_gpu(x, weight, bias)
    if x.dim() != 3:
        raise ValueError("x must be [batch, seq_len, hidden_size]")
    d = x.shape[-1]
    w2 = weight.detach().reshape(weight.shape[0], -1).to(x.dtype).contiguous()       # nn.Conv1d keeps [D, 1, W]
    if w2.shape[0] != d:
        raise ValueError(f"convolution has {w2.shape[0]} channels, the input {d}")
    b1 = bias.detach().to(x.dtype).contiguous() if bias is not None else None
    return dev, w2, b1


def short_conv(x, weight, bias=None, activation=True, cache=None):
    """Causal depthwise convolution (+ SiLU) of x [B, T, D] with weight [D, 1, W] / [D, W]; cache [B, D, W] (x.dtype,
    contiguous), when given, receives the last W inputs."""
    lib = L.load()
    dev, w2, b1 = _conv_args(x, weight, bias)
    b, t, d = x.shape
    xc = x.contiguous()
    y = torch.empty_like(xc)
    if cache is not None and not (cache.shape == (b, d, w2.shape[1]) and cache.dtype == x.dtype and cache.is_contiguous()
                                  and cache.device == dev):
        raise L.MMFError(f"short_conv: the cache must be a contiguous [{b}, {d}, {w2.shape[1]}] {x.dtype} tensor on {dev}")
    with torch.cuda.device(dev):
        L.check(lib.mmf_short_conv_fwd(xc.data_ptr(), w2.data_ptr(), L.ptr(b1), y.data_ptr(), L.ptr(cache), b, t, d, w2.shape[1],
                                       1 if activation else 0, L.dtype_id(x.dtype), L.stream()), "mmf_short_conv_fwd")
    return y


def short_conv_step(x, weight, bias, cache, activation=True):
    """One token: x [B, D]; the cache [B, D, W] is updated in place; returns y [B, D]."""
    lib = L.load()
    dev, w2, b1 = _conv_args(x.unsqueeze(1), weight, bias)
    b, d = x.shape
    if not (cache.shape == (b, d, w2.shape[1]) and cache.dtype == x.dtype and cache.is_contiguous() and cache.device == dev):
        raise L.MMFError(f"short_conv_step: the cache must be a contiguous [{b}, {d}, {w2.shape[1]}] {x.dtype} tensor on {dev}")
    xc = x.contiguous()
    y = torch.empty_like(xc)
    with torch.cuda.device(dev):
        L.check(lib.mmf_short_conv_step(xc.data_ptr(), w2.data_ptr(), L.ptr(b1), cache.data_ptr(), y.data_ptr(), b, d, w2.shape[1],
                                        1 if activation else 0, L.dtype_id(x.dtype), L.stream()), "mmf_short_conv_step")
    return y


def short_conv_bwd(x, weight, bias, dy, activation=True):
    """Gradients of short_conv: (dx [B, T, D] x.dtype, dweight [D, W] fp32, dbias [D] fp32)."""
    lib = L.load()
    dev, w2, b1 = _conv_args(x, weight, bias)
    b, t, d = x.shape
    w = w2.shape[1]
    xc, dyc = x.contiguous(), dy.contiguous()
    dx = torch.empty_like(xc)
    dpre = torch.empty(b, t, d, dtype=torch.float32, device=dev)
    part = torch.empty(lib.mmf_short_conv_bwd_groups(b * t), (w + 1) * d, dtype=torch.float32, device=dev)
    dwb = torch.empty((w + 1) * d, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        L.check(lib.mmf_short_conv_bwd(xc.data_ptr(), w2.data_ptr(), L.ptr(b1), dyc.data_ptr(), dx.data_ptr(), dpre.data_ptr(),
                                       part.data_ptr(), dwb.data_ptr(), b, t, d, w, 1 if activation else 0, L.dtype_id(x.dtype),
                                       L.stream()), "mmf_short_conv_bwd")
    return dx, dwb[:w * d].view(w, d).t(), dwb[w * d:]
