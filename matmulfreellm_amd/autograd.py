"""Training side: torch.autograd.Functions over the HIP forward and backward kernels.

Each Function mirrors one of the reference's autograd Functions:
  BitLinearFn              LayerNormLinearQuantFn        mmfreelm/ops/fusedbitnet.py:416-510
  RMSNormFn                LayerNormFn (RMS form)        mmfreelm/modules/layernorm.py:445-531
  RMSNormSwishGateFn       LayerNormFn (gated)           mmfreelm/modules/fused_norm_gate.py:420-500
  SwiGLUFn                 SwiGLUFunction                mmfreelm/modules/activations.py:143-175
  FusedRecurrentHGRNFn     FusedRecurrentHGRNFunction    mmfreelm/ops/hgrn/recurrent_fuse.py:136-173
  ChunkHGRNFn              ChunkHGRNFunction             mmfreelm/ops/hgrn/chunk.py:223-284
  HGRNGateFn               the elementwise ops of mmfreelm/layers/hgrn_bit.py:113-120, differentiated as one op
  CrossEntropyFn           CrossEntropyLossFunction      mmfreelm/modules/fused_cross_entropy.py:163-310

The forward values are those of the inference kernels (same launches); the backward kernels live in csrc/backward.hip.
The two dense products of a BitLinear's backward (dout @ W_q and dout^T @ y_q, fusedbitnet.py:474, :498) are plain
library GEMMs (torch.matmul).  Modules pick these Functions when gradients are enabled and an input or parameter
requires one (`needs_grad`); otherwise they keep the fused inference launches.
"""
import torch

from . import _lib as L
from . import functional as F_


def needs_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def module_needs_grad(module, *inputs) -> bool:
    """The rule every module uses to pick the differentiable path: gradients are enabled and an input or one of the module's
    parameters requires one -- whatever module.training says (the reference differentiates in eval mode too)."""
    return torch.is_grad_enabled() and (any(t is not None and t.requires_grad for t in inputs)
                                        or any(p.requires_grad for p in module.parameters()))


def _2d(t):
    return t.reshape(-1, t.shape[-1])


def _rows_ld(t):
    """[rows, K] view and its row stride; copies only if the last dimension is strided."""
    t2 = _2d(t)
    if t2.stride(-1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < t2.shape[1]):
        t2 = t2.contiguous()
    return t2, (t2.stride(0) if t2.shape[0] > 1 else t2.shape[1])


def _norm_bwd(mode, xs, gate, weight, dy, dres, eps, want_y=False):
    """Launch mmf_rmsnorm_bwd; returns (dx, dgate, y_quant, dweight)."""
    lib = L.load()
    dev = xs.device
    x2, ldx = _rows_ld(xs)
    dy2, lddy = _rows_ld(dy if dy.dtype == x2.dtype else dy.to(x2.dtype))
    m, k = x2.shape
    g2, ldg = _rows_ld(gate) if gate is not None else (None, 0)
    dr2 = _2d(dres).to(x2.dtype).contiguous() if dres is not None else None
    dx = torch.empty(m, k, dtype=x2.dtype, device=dev)
    dgate = torch.empty(m, k, dtype=x2.dtype, device=dev) if mode == 1 else None
    yq = torch.empty(m, k, dtype=x2.dtype, device=dev) if want_y else None
    w = weight.detach() if weight is not None else None
    if w is not None and w.dtype not in (torch.float32, x2.dtype):
        w = w.float()
    dw = torch.empty_like(w) if w is not None else None
    part = torch.empty(lib.mmf_backward_groups(m), k, dtype=torch.float32, device=dev) if w is not None else None
    with torch.cuda.device(dev):
        L.check(lib.mmf_rmsnorm_bwd(mode, x2.data_ptr(), ldx, L.ptr(g2), ldg, L.ptr(w), dy2.data_ptr(), lddy, L.ptr(dr2),
                                    dx.data_ptr(), L.ptr(dgate), L.ptr(yq), L.ptr(part), L.ptr(dw), m, k, eps,
                                    L.dtype_id(x2.dtype), L.dtype_id(w.dtype) if w is not None else 0, L.stream()),
                "mmf_rmsnorm_bwd")
    if dw is not None and weight is not None and dw.dtype != weight.dtype:
        dw = dw.to(weight.dtype)
    return dx, dgate, yq, dw


class RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, residual, eps, prenorm, residual_in_fp32):
        with torch.no_grad():
            if residual is not None or prenorm:
                y, res_out = F_.rmsnorm(x, weight, residual=residual, eps=eps, prenorm=True, residual_in_fp32=residual_in_fp32)
            else:
                y, res_out = F_.rmsnorm(x, weight, eps=eps), x
        ctx.save_for_backward(res_out, weight)
        ctx.eps, ctx.has_res, ctx.prenorm, ctx.x_dtype, ctx.shape = eps, residual is not None, prenorm, x.dtype, x.shape
        ctx.res_dtype = residual.dtype if residual is not None else None
        return (y, res_out) if prenorm else y

    @staticmethod
    def backward(ctx, dy, *rest):
        xs, weight = ctx.saved_tensors
        dres = rest[0] if (ctx.prenorm and rest and rest[0] is not None) else None
        dx, _, _, dw = _norm_bwd(0, xs, None, weight, dy.contiguous(), dres, ctx.eps)
        dx = dx.reshape(ctx.shape)
        dres_in = dx.to(ctx.res_dtype) if ctx.has_res else None
        return dx.to(ctx.x_dtype), dw, dres_in, None, None, None


class RMSNormSwishGateFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, o, weight, eps):
        with torch.no_grad():
            y = F_.rmsnorm_swishgate(x, o, weight, eps=eps)
        ctx.save_for_backward(x, o, weight)
        ctx.eps = eps
        return y

    @staticmethod
    def backward(ctx, dy):
        x, o, weight = ctx.saved_tensors
        dx, do, _, dw = _norm_bwd(1, x, o, weight, dy.contiguous(), None, ctx.eps)
        return dx.reshape(x.shape), do.reshape(o.shape), dw, None


class BitLinearFn(torch.autograd.Function):
    """RMSNorm -> int8 absmax quantiser -> ternary weights, straight-through gradients (fusedbitnet.py:416-510)."""

    @staticmethod
    def forward(ctx, x, norm_weight, weight, bias, eps, residual, prenorm, residual_in_fp32, pw):
        with torch.no_grad():
            if pw is None:
                pw = F_.ternarize_pack(weight)
            if residual is not None or prenorm:
                out, res_out = F_.bitlinear(x, norm_weight, pw, bias=bias, eps=eps, residual=residual, prenorm=True,
                                            residual_in_fp32=residual_in_fp32)
            else:
                out, res_out = F_.bitlinear(x, norm_weight, pw, bias=bias, eps=eps), x
        ctx.save_for_backward(res_out, norm_weight)
        ctx.pw, ctx.eps, ctx.has_res, ctx.prenorm, ctx.has_bias = pw, eps, residual is not None, prenorm, bias is not None
        ctx.w_dtype, ctx.x_dtype, ctx.shape = weight.dtype, x.dtype, x.shape
        ctx.res_dtype = residual.dtype if residual is not None else None
        ctx.bias_dtype = bias.dtype if bias is not None else None
        return (out, res_out) if prenorm else out

    @staticmethod
    def backward(ctx, dout, *rest):
        xs, norm_weight = ctx.saved_tensors
        pw = ctx.pw
        dres = rest[0] if (ctx.prenorm and rest and rest[0] is not None) else None
        d2 = _2d(dout).contiguous()
        # de-quantised ternary weights [N, K] in the activation dtype: t * wdeq
        wq = F_.unpack_ternary(pw).to(d2.dtype) * pw.wdeq.to(d2.dtype)
        dy = d2 @ wq                                                  # fusedbitnet.py:474
        dx, _, yq, dnw = _norm_bwd(2, xs, None, norm_weight, dy, dres, ctx.eps, want_y=True)
        dw = (d2.t() @ yq.to(d2.dtype)).to(ctx.w_dtype)              # fusedbitnet.py:498
        dbias = d2.sum(0).to(ctx.bias_dtype) if ctx.has_bias else None
        dx = dx.reshape(ctx.shape)
        dres_in = dx.to(ctx.res_dtype) if ctx.has_res else None
        return dx.to(ctx.x_dtype), dnw, dw, dbias, None, dres_in, None, None, None


class SwiGLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, y):
        with torch.no_grad():
            out = F_.swiglu(x, y)
        ctx.save_for_backward(x, y)
        return out

    @staticmethod
    def backward(ctx, g):
        x, y = ctx.saved_tensors
        lib = L.load()
        x2, ldx = _rows_ld(x)
        y2, ldy = _rows_ld(y)
        g2, ldg = _rows_ld(g)
        rows, cols = x2.shape
        dx = torch.empty(rows, cols, dtype=x.dtype, device=x.device)
        dy = torch.empty(rows, cols, dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            L.check(lib.mmf_swiglu_bwd(x2.data_ptr(), ldx, y2.data_ptr(), ldy, g2.data_ptr(), ldg, dx.data_ptr(), cols,
                                       dy.data_ptr(), cols, rows, cols, L.dtype_id(x.dtype), L.stream()), "mmf_swiglu_bwd")
        return dx.reshape(x.shape), dy.reshape(y.shape)


class HGRNGateFn(torch.autograd.Function):
    """(i, f) -> (x, g) of mmfreelm/layers/hgrn_bit.py:113-120 as one differentiable op."""

    @staticmethod
    def forward(ctx, i, f, lower_bound, mask):
        with torch.no_grad():
            x, g = F_.hgrn_gate(i, f, lower_bound, mask)
        ctx.save_for_backward(i, f, lower_bound, mask)
        return x, g

    @staticmethod
    def backward(ctx, gx, gg):
        i, f, lb, mask = ctx.saved_tensors
        lib = L.load()
        dev = i.device
        d = i.shape[-1]
        i2, ldi = _rows_ld(i)
        f2, ldf = _rows_ld(f)
        rows = i2.shape[0]
        gx2 = _2d(gx).to(i.dtype).contiguous() if gx is not None else torch.zeros(rows, d, dtype=i.dtype, device=dev)
        gg2 = _2d(gg).to(i.dtype).contiguous() if gg is not None else torch.zeros(rows, d, dtype=i.dtype, device=dev)
        di = torch.empty(rows, d, dtype=i.dtype, device=dev)
        df = torch.empty(rows, d, dtype=i.dtype, device=dev)
        lbf = lb.detach().float().contiguous() if lb is not None else None
        dlb = torch.empty(d, dtype=torch.float32, device=dev) if lb is not None else None
        part = torch.empty(lib.mmf_backward_groups(rows), d, dtype=torch.float32, device=dev) if lb is not None else None
        mk = F_._mask_rows(mask, rows, dev) if mask is not None else None
        with torch.cuda.device(dev):
            L.check(lib.mmf_hgrn_gate_bwd(i2.data_ptr(), ldi, f2.data_ptr(), ldf, L.ptr(lbf), L.ptr(mk), gx2.data_ptr(),
                                          gg2.data_ptr(), di.data_ptr(), d, df.data_ptr(), d, L.ptr(part), L.ptr(dlb), rows, d,
                                          L.dtype_id(i.dtype), L.stream()), "mmf_hgrn_gate_bwd")
        return di.reshape(i.shape), df.reshape(f.shape), (dlb.to(lb.dtype) if lb is not None else None), None


def _scan_bwd(g, o, do, h0, log_gates):
    lib = L.load()
    b, h, t, d = g.shape
    gc, oc, dc = g.contiguous(), o.contiguous(), do.to(g.dtype).contiguous()
    dx, dg = torch.empty_like(gc), torch.empty_like(gc)
    h0f = h0.detach().reshape(b * h, d).float().contiguous() if h0 is not None else None
    with torch.cuda.device(g.device):
        L.check(lib.mmf_hgrn_recurrent_bwd(gc.data_ptr(), oc.data_ptr(), dc.data_ptr(), L.ptr(h0f), dx.data_ptr(), dg.data_ptr(),
                                           b * h, t, d, 1 if log_gates else 0, L.dtype_id(g.dtype), L.stream()),
                "mmf_hgrn_recurrent_bwd")
    return dx, dg


class FusedRecurrentHGRNFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, g, initial_state, output_final_state):
        with torch.no_grad():
            o, ht = F_.hgrn_recurrent(x, g, initial_state, output_final_state)
        ctx.save_for_backward(g, o, initial_state)
        if ht is not None:
            ctx.mark_non_differentiable(ht)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht=None):
        g, o, h0 = ctx.saved_tensors
        dx, dg = _scan_bwd(g, o, do, h0, False)
        return dx, dg, None, None


class ChunkHGRNFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, g, initial_state, output_final_state, chunk_size):
        with torch.no_grad():
            o, ht = F_.hgrn_chunk(x, g, initial_state, output_final_state, chunk_size)
        ctx.save_for_backward(g, o, initial_state)
        if ht is not None:
            ctx.mark_non_differentiable(ht)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht=None):
        g, o, h0 = ctx.saved_tensors
        dx, dg = _scan_bwd(g, o, do, h0, True)
        return dx, dg, None, None, None


class CrossEntropyFn(torch.autograd.Function):
    """Per-row losses (and z-losses) of [rows, V] logits; mmfreelm/modules/fused_cross_entropy.py:163-310 on one device."""

    @staticmethod
    def forward(ctx, logits, labels, smoothing, logit_scale, lse_square_scale, ignore_index, inplace_backward):
        lib = L.load()
        dev = L.require_gpu(logits, labels)
        if logits.dim() != 2 or labels.shape != (logits.shape[0],):
            raise ValueError("logits [rows, V] and one label per row")
        lg = logits if logits.stride(-1) == 1 else logits.contiguous()
        lab = labels.to(torch.int64).contiguous()
        rows, v = lg.shape
        loss = torch.empty(rows, dtype=torch.float32, device=dev)
        lse = torch.empty(rows, dtype=torch.float32, device=dev)
        z = torch.empty(rows, dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            L.check(lib.mmf_cross_entropy_train_fwd(lg.data_ptr(), lg.stride(0), lab.data_ptr(), int(ignore_index), float(smoothing),
                                                    float(logit_scale), float(lse_square_scale), loss.data_ptr(), lse.data_ptr(),
                                                    z.data_ptr(), rows, v, L.dtype_id(lg.dtype), L.stream()),
                    "mmf_cross_entropy_train_fwd")
        ctx.save_for_backward(lg, lab, lse)
        ctx.args = (float(smoothing), float(logit_scale), float(lse_square_scale), int(ignore_index), bool(inplace_backward))
        ctx.mark_non_differentiable(z)
        return loss, z

    @staticmethod
    def backward(ctx, dloss, dz=None):
        lg, lab, lse = ctx.saved_tensors
        smoothing, logit_scale, lse_square_scale, ignore_index, inplace = ctx.args
        lib = L.load()
        rows, v = lg.shape
        dlogits = lg if inplace else torch.empty_like(lg)
        dl = dloss.to(torch.float32).contiguous()
        with torch.cuda.device(lg.device):
            L.check(lib.mmf_cross_entropy_train_bwd(lg.data_ptr(), lg.stride(0), lab.data_ptr(), ignore_index, lse.data_ptr(),
                                                    dl.data_ptr(), smoothing, logit_scale, lse_square_scale, dlogits.data_ptr(),
                                                    dlogits.stride(0), rows, v, L.dtype_id(lg.dtype), L.stream()),
                    "mmf_cross_entropy_train_bwd")
        return dlogits, None, None, None, None, None, None


class FusedCrossEntropyLoss(torch.nn.Module):
    """mmfreelm/modules/fused_cross_entropy.py:323-398 (one device: no process_group)."""

    def __init__(self, ignore_index=-100, reduction="mean", label_smoothing=0.0, logit_scale=1.0, lse_square_scale=0.0,
                 inplace_backward=False, process_group=None, return_z_loss=False):
        super().__init__()
        if reduction not in ("mean", "none", "sum"):
            raise NotImplementedError("Only support reduction = 'mean' or 'none' or 'sum'")
        if process_group is not None:
            raise NotImplementedError("the vocabulary-parallel loss needs a process group; this build runs on one GPU")
        self.ignore_index, self.reduction, self.label_smoothing = ignore_index, reduction, label_smoothing
        self.logit_scale, self.lse_square_scale = logit_scale, lse_square_scale
        self.inplace_backward, self.return_z_loss = inplace_backward, return_z_loss

    def forward(self, input, target):
        loss, z_loss = CrossEntropyFn.apply(input, target, self.label_smoothing, self.logit_scale, self.lse_square_scale,
                                            self.ignore_index, self.inplace_backward)
        if self.reduction == "mean":
            n = (target != self.ignore_index).sum()
            loss, z_loss = loss.sum() / n, z_loss.sum() / n
        elif self.reduction == "sum":
            loss, z_loss = loss.sum(), z_loss.sum()
        return (loss, z_loss) if self.return_z_loss else loss


class ShortConvFn(torch.autograd.Function):
    """ShortConvolution.forward over whole sequences (mmfreelm/modules/convolution.py:98-131) as one differentiable op."""

    @staticmethod
    def forward(ctx, x, weight, bias, activation):
        with torch.no_grad():
            y = F_.short_conv(x, weight, bias, activation)
        ctx.save_for_backward(x, weight, bias)
        ctx.activation = activation
        return y

    @staticmethod
    def backward(ctx, g):
        x, weight, bias = ctx.saved_tensors
        dx, dw, db = F_.short_conv_bwd(x, weight, bias, g, ctx.activation)
        dweight = dw.reshape(weight.shape).to(weight.dtype) if ctx.needs_input_grad[1] else None
        dbias = db.to(bias.dtype) if (bias is not None and ctx.needs_input_grad[2]) else None
        return dx, dweight, dbias, None
