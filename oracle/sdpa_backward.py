"""TEST INFRASTRUCTURE ONLY -- gradients of the reference CPU attention op, restated in numpy.

The reference has no backward kernel for attention: its operator is a composition of taped ops
(crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269) and the gradient is what walking that tape gives
(crates/incin-backends/src/cpu/tape.rs:149-176).  Node by node, in reverse:

  out = attn @ v          matmul: grad_lhs = grad_out @ rhs^T, grad_rhs = lhs^T @ grad_out
                          (cpu/ops/matmul.rs:264-281; batch axes broadcast, gradients summed back over broadcast
                          axes by tape::unbroadcast, cpu/tape.rs:247-280)
  attn = exp(ls)          d ls = d attn * attn                              (FloatOps::exp)
  ls = log_softmax(x)     composed of max_keepdim, sub, exp, sum_keepdim, log, sub (cpu/ops/elementwise.rs:1062-1077);
                          the chain collapses to  d x = d ls - exp(ls) * sum_j(d ls)   (the max term cancels)
  x = scaled + mask       d scaled = d x                                    (NumericOps::add; the mask is a constant here)
  scaled = scores * s     d scores = d scaled * (f32) s                     (mul_scalar_float, elementwise.rs:390-419)
  scores = q @ k^T        d q = d scores @ k,  d k = d scores^T @ q         (matmul + transpose backward)

Evaluated here in float64 from float32 operands (the reference runs the same formulas in f32 with f64-accumulated
products); results are returned as float64.  `matmul_backward` is the single-node rule on its own, pinned by the
reference's hand-computed case (cpu/ops/matmul.rs:728-770)."""
import numpy as np


def matmul_backward(lhs, rhs, grad_out):
    """(grad_lhs, grad_rhs) of out = lhs @ rhs for 2-D operands."""
    lhs, rhs, grad_out = (np.asarray(x, np.float64) for x in (lhs, rhs, grad_out))
    return grad_out @ rhs.T, lhs.T @ grad_out


def _unbroadcast(g, shape):
    """Sum `g` back to `shape` (right-aligned NumPy broadcast), as tape::unbroadcast does."""
    g = g.sum(axis=tuple(range(g.ndim - len(shape)))) if g.ndim > len(shape) else g
    for ax, n in enumerate(shape):
        if n == 1 and g.shape[ax] != 1:
            g = g.sum(axis=ax, keepdims=True)
    return g


def additive_mask(Sq, Skv, batch_shape, causal=False, kv_lens=None):
    """The 0 / -inf mask that `causal` (key j > i + Skv - Sq) and `kv_lens` (key j >= len, lens broadcastable to
    batch_shape) stand for, shape batch_shape + [Sq, Skv]."""
    m = np.zeros(tuple(batch_shape) + (Sq, Skv), np.float64)
    if causal:
        m = m + np.triu(np.full((Sq, Skv), -np.inf), 1 + Skv - Sq)
    if kv_lens is not None:
        lens = np.broadcast_to(np.asarray(kv_lens), batch_shape)
        m = m + np.where(np.arange(Skv) < lens[..., None, None], 0.0, -np.inf)
    return m


def sdpa_forward_f64(q, k, v, mask=None, scale=None):
    """softmax(q k^T s + mask) v in float64 and the probabilities, batch axes broadcast."""
    q, k, v = (np.asarray(x, np.float64) for x in (q, k, v))
    s = float(np.float32(1.0 / np.sqrt(q.shape[-1]) if scale is None else scale))
    x = np.matmul(q, np.swapaxes(k, -1, -2)) * s
    if mask is not None:
        x = x + np.asarray(mask, np.float64)
    with np.errstate(invalid="ignore"):
        mx = x.max(-1, keepdims=True)
        e = np.exp(x - mx)
        p = e / e.sum(-1, keepdims=True)
    return np.matmul(p, v), p, s


def sdpa_backward(q, k, v, grad_out, mask=None, scale=None, causal=False, kv_lens=None):
    """(dq, dk, dv) of the reference composition for upstream gradient `grad_out` [..., Sq, Dv].

    `causal` / `kv_lens` are folded into the additive mask first (the reference knows one mask tensor).  Rows whose
    keys are all masked give NaN, as the forward does."""
    q, k, v, go = (np.asarray(x, np.float64) for x in (q, k, v, grad_out))
    Sq, Skv = q.shape[-2], k.shape[-2]
    bshape = np.broadcast_shapes(q.shape[:-2], k.shape[:-2], v.shape[:-2])
    if causal or kv_lens is not None:
        extra = additive_mask(Sq, Skv, bshape, causal, kv_lens)
        mask = extra if mask is None else np.asarray(mask, np.float64) + extra
    out, p, s = sdpa_forward_f64(q, k, v, mask, scale)
    dv = np.matmul(np.swapaxes(p, -1, -2), go)                     # attn^T @ grad_out
    dp = _unbroadcast(np.matmul(go, np.swapaxes(v, -1, -2)), p.shape)      # grad_out @ v^T, back to attn's shape
    dls = dp * p
    dx = dls - p * dls.sum(-1, keepdims=True)
    # the mask's add may have widened the scores (more batch axes, or rows where q has one): its gradient rule sums
    # those back to the shape of q k^T before the scale and the first product's rules apply (cpu/tape.rs:243-265)
    scores_shape = tuple(np.broadcast_shapes(q.shape[:-2], k.shape[:-2])) + (Sq, Skv)
    dscores = _unbroadcast(dx, scores_shape) * s
    dq = np.matmul(dscores, k)
    dk = np.matmul(np.swapaxes(dscores, -1, -2), q)
    return _unbroadcast(dq, q.shape), _unbroadcast(dk, k.shape), _unbroadcast(dv, v.shape)


def logsumexp(q, k, mask=None, scale=None, causal=False, kv_lens=None):
    """Natural-log normaliser of every row, log sum_j exp(x_ij): what a fused backward needs from the forward."""
    q, k = np.asarray(q, np.float64), np.asarray(k, np.float64)
    Sq, Skv = q.shape[-2], k.shape[-2]
    bshape = np.broadcast_shapes(q.shape[:-2], k.shape[:-2])
    if causal or kv_lens is not None:
        extra = additive_mask(Sq, Skv, bshape, causal, kv_lens)
        mask = extra if mask is None else np.asarray(mask, np.float64) + extra
    s = float(np.float32(1.0 / np.sqrt(q.shape[-1]) if scale is None else scale))
    x = np.matmul(q, np.swapaxes(k, -1, -2)) * s
    if mask is not None:
        x = x + mask
    with np.errstate(invalid="ignore", divide="ignore"):
        mx = x.max(-1, keepdims=True)
        return (mx + np.log(np.exp(x - mx).sum(-1, keepdims=True)))[..., 0]
