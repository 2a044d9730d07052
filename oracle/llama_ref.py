"""CPU oracle, part 2: the llama2-style transformer of the reference's
test/llama.py, forward and reverse-mode gradient, in numpy.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.

Three layers of restatement, each checked against the one before it:

1. `forward_step` follows test/llama.py:35-238 line by line (single token,
   vectors of length `dim`, KV cache append, per-head softmax).  It is the
   literal reference algorithm.
2. The batched / causal functions (`rmsnorm_fwd`, `rope_fwd`, `attention_fwd`,
   `swiglu_fwd`, `linear_fwd`, `layer_fwd`, `model_fwd`) are the same maths over
   activations [B, S, D]; tests replay `forward_step` for pos = 0..S-1 with a
   real cache and require equality.
3. The closed-form adjoints (`*_bwd`) are what the fused HIP kernels implement.
   They are checked against `*_bwd_by_rules`, which chain the reference's
   per-op rules (oracle/ad_rules.py, pinned by the reference's lit vectors) in
   the exact op order test/llama.py traces, against central finite differences
   in float64, and against an independent torch.autograd restatement.

Parity status: every function here is pinned by at least one of: the step-form
replay, the rule-chained adjoint, finite differences, torch.autograd, or a
closed-form special case (tests/test_oracle_*.py).  The cross-entropy functions
(section 4b) have no call site in the reference; they are pinned by closed forms,
scipy's logsumexp, torch's float64 cross_entropy and finite differences.  What cannot be pinned
without running the reference: the bit pattern of XLA-CPU's compiled result
(summation order, 1/sqrt -> rsqrt rewrite); the reference's own test tolerates
atol = rtol = 1e-3 there (test/llama.py:318-319) - "parity unpinned" below
that tolerance for XLA codegen only.
"""
import numpy as np

from . import ad_rules as R

EPS = 1e-5          # test/llama.py:9
ROPE_THETA = 10000  # test/llama.py:130


# ---------------------------------------------------------------------------
# 1. Literal single-token step (test/llama.py)
# ---------------------------------------------------------------------------

def rmsnorm(x, weight):
    """test/llama.py:6-10."""
    ss = 1 / np.sqrt(x.dot(x) / x.shape[0] + 1e-5)
    return weight * x * ss


def softmax(x):
    """test/llama.py:13-18 (global max of the vector, python sum)."""
    max_val = np.max(x)
    x = np.exp(x - max_val)
    return x / sum(x)


def sigmoid(x):
    """test/llama.py:21-24."""
    return 1 / (1 + np.exp(-x))


def silu(x):
    """test/llama.py:27-28."""
    return x * sigmoid(x)


def forward_step(x, config, weights, key_cache, value_cache, return_caches=False):
    """test/llama.py:35-238.  `key_cache`/`value_cache`: (n_layers, pos, kv_dim);
    the token being processed sits at position `pos`.  Returns the final
    RMSNorm of the residual stream (the logits matmul is commented out in the
    reference, :236)."""
    pos = key_cache.shape[1]
    n_layers = config["n_layers"]
    n_heads = config["n_heads"]
    dim = config["dim"]
    n_kv_heads = config["n_kv_heads"]
    head_size = dim // n_heads
    kv_mul = n_heads // n_kv_heads
    kv_dim = dim // n_heads * n_kv_heads
    wq, wk, wv, wo = weights["wq"], weights["wk"], weights["wv"], weights["wo"]
    w1, w2, w3 = weights["w1"], weights["w2"], weights["w3"]

    toconv = []
    for i in range(0, dim, 2):                                  # :127-135
        freq = 1 / np.power(10000.0, (i % head_size) / head_size)
        val = pos * freq
        fcr, fci = np.cos(val), np.sin(val)
        toconv.append(np.array([[fcr, -fci], [fci, fcr]]))
    toconv2 = toconv[: kv_dim // 2] + [np.eye(2)] * (dim // 2 - kv_dim // 2)
    toconv = np.array(toconv)
    toconv2 = np.array(toconv2)

    keys2, values2 = [], []
    x = np.array(x, copy=True)
    for i in range(n_layers):
        xb = rmsnorm(x, weights["rms_att_weight"][i, :])        # :145
        q = wq[i] @ xb                                          # :149-157
        k = wk[i] @ xb
        v = wv[i] @ xb
        q_tmp = np.reshape(q, (dim // 2, 2))
        k_tmp = np.reshape(k, (dim // 2, 2))
        k = np.reshape(np.einsum("ijk,ik -> ij", toconv2, k_tmp), (dim,))   # :167
        q = np.reshape(np.einsum("ijk,ik -> ij", toconv, q_tmp), (dim,))    # :168
        key_cache_l = np.append(key_cache[i], np.reshape(k, (1, dim)), axis=0)     # :170-173
        value_cache_l = np.append(value_cache[i], np.reshape(v, (1, dim)), axis=0)
        keys2.append(key_cache_l)
        values2.append(value_cache_l)
        xbs2 = []
        for h in range(n_heads):                                # :178-206
            q2 = q[head_size * h: head_size * (h + 1)]
            key_index = h // kv_mul
            att = np.einsum("ij,j->i", key_cache_l[:, key_index * head_size:(key_index + 1) * head_size], q2)
            att = att / np.sqrt(head_size)
            att = softmax(att)
            x_tmp = np.einsum("ij,i->j", value_cache_l[:, key_index * head_size:(key_index + 1) * head_size], att)
            xbs2.append(x_tmp)
        xb = np.concatenate(xbs2, axis=None)
        x = x + wo[i] @ xb                                      # :211-215
        xb = rmsnorm(x, weights["rms_ffn_weight"][i, :])        # :219
        hb = w1[i] @ xb                                         # :224-231
        hb2 = w3[i] @ xb
        hb = silu(hb) * hb2
        x = x + w2[i] @ hb                                      # :233
    x = rmsnorm(x, weights["rms_final_weight"])                 # :235
    if return_caches:
        return x, np.array(keys2), np.array(values2)
    return x


# ---------------------------------------------------------------------------
# 2. Batched building blocks, forward
# ---------------------------------------------------------------------------

def rmsnorm_fwd(x, gamma, eps=EPS):
    """y = gamma * x * rsqrt(mean(x^2) + eps) over the last dim (llama.py:6-10)."""
    r = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return gamma * x * r


def rope_angles(S, head_dim, theta=ROPE_THETA, pos0=0, dtype=np.float64):
    """cos/sin tables [S, head_dim/2] for positions pos0..pos0+S-1
    (llama.py:127-133: freq_j = theta^(-(2j)/head_dim), angle = pos * freq)."""
    j = np.arange(0, head_dim, 2, dtype=np.float64)
    freq = 1.0 / np.power(float(theta), j / head_dim)
    pos = np.arange(pos0, pos0 + S, dtype=np.float64)[:, None]
    ang = pos * freq[None, :]
    return np.cos(ang).astype(dtype), np.sin(ang).astype(dtype)


def rope_fwd(x, cos, sin, inverse=False):
    """x: [B, S, h, d]; rotates adjacent pairs (2p, 2p+1) by +angle (llama.py:135,
    161-168), or by -angle when `inverse` (the adjoint: transpose of the 2x2)."""
    x0, x1 = x[..., 0::2], x[..., 1::2]
    c = cos[None, :, None, :]
    s = sin[None, :, None, :]
    if inverse:
        s = -s
    y = np.empty_like(x)
    y[..., 0::2] = c * x0 - s * x1
    y[..., 1::2] = s * x0 + c * x1
    return y


def linear_fwd(x, w):
    """Y[..., out] = X[..., in] . W[out, in]^T  (llama.py:149: `wq[i] @ xb`)."""
    return x @ w.T


def attention_fwd(q, k, v, scale=None, causal=True):
    """q, k, v: [B, h, S, d].  Scores = (q . k) * scale applied after the dot
    (llama.py:190-196), softmax over keys 0..t for query t (the cache holds
    only positions <= pos), out = sum_t att[t] v[t] (llama.py:200-204).
    Returns (o, lse) with lse = log sum exp of the scaled scores per query."""
    B, h, S, d = q.shape
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    if causal:
        mask = np.tril(np.ones((S, k.shape[2]), dtype=bool), k=k.shape[2] - S)
        s = np.where(mask, s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    p = np.exp(s - m)
    l = np.sum(p, axis=-1, keepdims=True)
    p = p / l
    o = np.einsum("bhqk,bhkd->bhqd", p, v)
    lse = (m + np.log(l))[..., 0]
    return o, lse


def swiglu_fwd(a, b):
    """g = a * sigmoid(a) * b  (llama.py:224-231, sigmoid spelled 1/(1+exp(-a)))."""
    return a * (1.0 / (1.0 + np.exp(-a))) * b


# ---------------------------------------------------------------------------
# 3. Closed-form adjoints (what the fused kernels implement)
# ---------------------------------------------------------------------------

def rmsnorm_bwd(x, gamma, dy, eps=EPS):
    """r = rsqrt(mean(x^2)+eps); g = dy*gamma;
    dx = r*g - x * r^3 * mean(g*x);  dgamma = sum_rows dy * x * r."""
    D = x.shape[-1]
    r = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    g = dy * gamma
    dx = r * g - x * (r ** 3) * (np.sum(g * x, axis=-1, keepdims=True) / D)
    dgamma = np.sum((dy * x * r).reshape(-1, D), axis=0)
    return dx, dgamma


def rope_bwd(dy, cos, sin):
    """Adjoint of the rotation = rotation by the negative angle."""
    return rope_fwd(dy, cos, sin, inverse=True)


def linear_bwd(x, w, dy):
    """dX = dY . W (NN), dW = dY^T . X (TN, reduced over all tokens)."""
    D_in = x.shape[-1]
    D_out = w.shape[0]
    dx = dy @ w
    dw = dy.reshape(-1, D_out).T @ x.reshape(-1, D_in)
    return dx, dw


def attention_bwd(q, k, v, do, scale=None, causal=True):
    """dV = P^T dO; dP = dO V^T; delta = rowsum(dO*O); dS = P*(dP - delta);
    dQ = dS K * scale; dK = dS^T Q * scale."""
    B, h, S, d = q.shape
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    if causal:
        mask = np.tril(np.ones((S, k.shape[2]), dtype=bool), k=k.shape[2] - S)
        s = np.where(mask, s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    p = np.exp(s - m)
    p = p / np.sum(p, axis=-1, keepdims=True)
    o = np.einsum("bhqk,bhkd->bhqd", p, v)
    dv = np.einsum("bhqk,bhqd->bhkd", p, do)
    dp = np.einsum("bhqd,bhkd->bhqk", do, v)
    delta = np.sum(do * o, axis=-1, keepdims=True)
    ds = p * (dp - delta)
    dq = np.einsum("bhqk,bhkd->bhqd", ds, k) * scale
    dk = np.einsum("bhqk,bhqd->bhkd", ds, q) * scale
    return dq, dk, dv


def swiglu_bwd(a, b, dg):
    """da = dg*b*s*(1 + a*(1-s)); db = dg*a*s, s = sigmoid(a)."""
    s = 1.0 / (1.0 + np.exp(-a))
    return dg * b * s * (1.0 + a * (1.0 - s)), dg * a * s


# ---------------------------------------------------------------------------
# 3b. The same adjoints obtained by chaining the reference's per-op rules in
#     the op order test/llama.py traces (vector form).  These tie the closed
#     forms above to the rule table that the lit vectors pin.
# ---------------------------------------------------------------------------

def rmsnorm_bwd_by_rules(x, weight, dy):
    """Reverse of llama.py:6-10:  t0 = x.x ; t1 = t0/n ; t2 = t1+eps ;
    t3 = sqrt(t2) ; ss = 1/t3 ; u = weight*x ; y = u*ss."""
    n = x.shape[0]
    t0 = x.dot(x)
    t1 = t0 / n
    t2 = t1 + 1e-5
    t3 = np.sqrt(t2)
    ss = 1.0 / t3
    u = weight * x
    # y = u * ss
    du, dss = R.vjp_multiply(u, ss, dy)
    dss = np.sum(dss)                       # ss is a scalar broadcast over the vector
    dweight, dx = R.vjp_multiply(weight, x, du)
    _, dt3 = R.vjp_divide(1.0, t3, dss)
    (dt2,) = R.vjp_sqrt(t2, dt3)
    dt1, _ = R.vjp_add(t1, 1e-5, dt2)
    dt0, _ = R.vjp_divide(t0, float(n), dt1)
    # t0 = x.x : dot_general with both operands = x (dot_general_3.mlir form)
    dx = dx + dt0 * x + dt0 * x
    return dx, dweight


def softmax_bwd_by_rules(x, dy):
    """Reverse of llama.py:13-18: m = max(x); z = x - m; e = exp(z);
    s = sum(e); y = e / s."""
    m = np.max(x)
    z = x - m
    e = np.exp(z)
    s = np.sum(e)
    de, ds = R.vjp_divide(e, s, dy)
    ds = np.sum(ds)
    (de2,) = R.vjp_reduce_add(e, 0, np.asarray(ds))
    de = de + de2
    (dz,) = R.vjp_exponential(z, de)
    dx, dm = R.vjp_subtract(x, m, dz)
    dm = np.sum(dm)
    (dx2,) = R.vjp_reduce_max(x, 0, np.asarray(dm))
    return dx + dx2


def silu_mul_bwd_by_rules(a, b, dg):
    """Reverse of llama.py:21-28,229-231: n = -a; e = exp(n); p = 1+e;
    s = 1/p; h = a*s; g = h*b."""
    n = -a
    e = np.exp(n)
    p = 1.0 + e
    s = 1.0 / p
    h = a * s
    dh, db = R.vjp_multiply(h, b, dg)
    da, ds = R.vjp_multiply(a, s, dh)
    _, dp = R.vjp_divide(1.0, p, ds)
    _, de = R.vjp_add(1.0, e, dp)
    (dn,) = R.vjp_exponential(n, de)
    (da2,) = R.vjp_negate(a, dn)
    return da + da2, db


# ---------------------------------------------------------------------------
# 4. Layer and model, batched
# ---------------------------------------------------------------------------

def _heads(x, n_heads):
    B, S, D = x.shape
    return x.reshape(B, S, n_heads, D // n_heads)


def layer_fwd(x, lw, n_heads, eps=EPS, theta=ROPE_THETA, pos0=0):
    """One decoder layer over x [B, S, D] (llama.py:144-233, batched/causal).
    lw: dict with rms_att_weight[D], wq/wk/wv/wo [D, D], rms_ffn_weight[D],
    w1/w3 [H, D], w2 [D, H].  Returns (y, cache-for-backward)."""
    B, S, D = x.shape
    d = D // n_heads
    cos, sin = rope_angles(S, d, theta, pos0, dtype=x.dtype)
    xb = rmsnorm_fwd(x, lw["rms_att_weight"], eps)
    q = linear_fwd(xb, lw["wq"])
    k = linear_fwd(xb, lw["wk"])
    v = linear_fwd(xb, lw["wv"])
    qr = rope_fwd(_heads(q, n_heads), cos, sin)
    kr = rope_fwd(_heads(k, n_heads), cos, sin)
    vh = _heads(v, n_heads)
    o, _ = attention_fwd(qr.transpose(0, 2, 1, 3), kr.transpose(0, 2, 1, 3),
                         vh.transpose(0, 2, 1, 3), 1.0 / np.sqrt(d), True)
    att = o.transpose(0, 2, 1, 3).reshape(B, S, D)
    x1 = x + linear_fwd(att, lw["wo"])
    xb2 = rmsnorm_fwd(x1, lw["rms_ffn_weight"], eps)
    a1 = linear_fwd(xb2, lw["w1"])
    a3 = linear_fwd(xb2, lw["w3"])
    g = swiglu_fwd(a1, a3)
    y = x1 + linear_fwd(g, lw["w2"])
    cache = dict(x=x, xb=xb, qr=qr, kr=kr, vh=vh, att=att, x1=x1, xb2=xb2,
                 a1=a1, a3=a3, g=g, cos=cos, sin=sin)
    return y, cache


def layer_bwd(dy, lw, cache, n_heads, eps=EPS):
    """Reverse of layer_fwd: returns (dx, dict of weight gradients)."""
    c = cache
    B, S, D = dy.shape
    d = D // n_heads
    gw = {}
    dg, gw["w2"] = linear_bwd(c["g"], lw["w2"], dy)
    da1, da3 = swiglu_bwd(c["a1"], c["a3"], dg)
    dxb2a, gw["w1"] = linear_bwd(c["xb2"], lw["w1"], da1)
    dxb2b, gw["w3"] = linear_bwd(c["xb2"], lw["w3"], da3)
    dx1n, gw["rms_ffn_weight"] = rmsnorm_bwd(c["x1"], lw["rms_ffn_weight"], dxb2a + dxb2b, eps)
    dx1 = dy + dx1n
    datt, gw["wo"] = linear_bwd(c["att"], lw["wo"], dx1)
    do = _heads(datt, n_heads).transpose(0, 2, 1, 3)
    dq, dk, dv = attention_bwd(c["qr"].transpose(0, 2, 1, 3), c["kr"].transpose(0, 2, 1, 3),
                               c["vh"].transpose(0, 2, 1, 3), do, 1.0 / np.sqrt(d), True)
    dq = rope_bwd(dq.transpose(0, 2, 1, 3), c["cos"], c["sin"]).reshape(B, S, D)
    dk = rope_bwd(dk.transpose(0, 2, 1, 3), c["cos"], c["sin"]).reshape(B, S, D)
    dv = dv.transpose(0, 2, 1, 3).reshape(B, S, D)
    dxb_q, gw["wq"] = linear_bwd(c["xb"], lw["wq"], dq)
    dxb_k, gw["wk"] = linear_bwd(c["xb"], lw["wk"], dk)
    dxb_v, gw["wv"] = linear_bwd(c["xb"], lw["wv"], dv)
    dxn, gw["rms_att_weight"] = rmsnorm_bwd(c["x"], lw["rms_att_weight"], dxb_q + dxb_k + dxb_v, eps)
    return dx1 + dxn, gw


LAYER_KEYS = ("rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3")


def _layer_weights(weights, i):
    return {k: weights[k][i] for k in LAYER_KEYS}


def model_fwd(x_or_tokens, weights, config, logits=False, eps=EPS, theta=ROPE_THETA):
    """Whole model over [B, S]: optional embedding gather (when the input is an
    integer token array and `token_embedding_table` is present; commented out
    in the reference, llama.py:109-113), n_layers decoder layers, final
    RMSNorm (:235) and, when `logits`, the `wcls` projection (:236)."""
    n_layers, n_heads = config["n_layers"], config["n_heads"]
    tokens = None
    if np.issubdtype(np.asarray(x_or_tokens).dtype, np.integer):
        tokens = np.asarray(x_or_tokens)
        x = weights["token_embedding_table"][tokens]
    else:
        x = x_or_tokens
    caches = []
    for i in range(n_layers):
        x, c = layer_fwd(x, _layer_weights(weights, i), n_heads, eps, theta)
        caches.append(c)
    xf = rmsnorm_fwd(x, weights["rms_final_weight"], eps)
    out = linear_fwd(xf, weights["wcls"]) if logits else xf
    return out, dict(tokens=tokens, caches=caches, x_last=x, xf=xf, logits=logits)


def model_bwd(dout, weights, config, fcache, eps=EPS):
    """Reverse of model_fwd: returns (dx or None, dict of weight gradients
    stacked per layer like the weights themselves)."""
    n_layers, n_heads = config["n_layers"], config["n_heads"]
    gw = {}
    if fcache["logits"]:
        dxf, gw["wcls"] = linear_bwd(fcache["xf"], weights["wcls"], dout)
    else:
        dxf = dout
    dx, gw["rms_final_weight"] = rmsnorm_bwd(fcache["x_last"], weights["rms_final_weight"], dxf, eps)
    per_layer = [None] * n_layers
    for i in reversed(range(n_layers)):
        dx, per_layer[i] = layer_bwd(dx, _layer_weights(weights, i), fcache["caches"][i], n_heads, eps)
    for k in LAYER_KEYS:
        gw[k] = np.stack([per_layer[i][k] for i in range(n_layers)])
    if fcache["tokens"] is not None:
        tab = weights["token_embedding_table"]
        g = np.zeros(tab.shape, dtype=dx.dtype)
        np.add.at(g, fcache["tokens"].reshape(-1), dx.reshape(-1, dx.shape[-1]))
        gw["token_embedding_table"] = g
        return None, gw
    return dx, gw


# ---------------------------------------------------------------------------
# 4b. Softmax cross-entropy on the logits.  The reference's llama test stops before
#     the classifier (test/llama.py:236 is commented out), so there is no reference
#     call site; the definition is the standard one (per token logsumexp(z) - z[t]),
#     built from the same softmax as test/llama.py:13-18.  Pinned by closed forms
#     (uniform logits give log V; shifting a row changes nothing; gradient rows sum
#     to zero), by scipy's logsumexp, by torch's float64 cross_entropy + autograd and
#     by central finite differences (tests/test_oracle_llama.py).
# ---------------------------------------------------------------------------

def cross_entropy_fwd(logits, targets):
    """(loss[...], lse[...]) for logits [..., V] and integer targets [...]; a target outside [0, V) masks its token."""
    z = np.asarray(logits, dtype=np.float64)
    t = np.asarray(targets)
    m = z.max(axis=-1, keepdims=True)                                     # test/llama.py:16 (max subtracted first)
    lse = (m + np.log(np.exp(z - m).sum(axis=-1, keepdims=True)))[..., 0]
    live = (t >= 0) & (t < z.shape[-1])
    picked = np.take_along_axis(z, np.where(live, t, 0)[..., None].astype(np.int64), axis=-1)[..., 0]
    return np.where(live, lse - picked, 0.0), lse


def cross_entropy_bwd(logits, targets, dloss):
    """dlogits = (softmax(z) - onehot(t)) * dloss."""
    z = np.asarray(logits, dtype=np.float64)
    t = np.asarray(targets)
    _, lse = cross_entropy_fwd(z, t)
    live = (t >= 0) & (t < z.shape[-1])
    p = np.exp(z - lse[..., None])
    onehot = (np.arange(z.shape[-1]) == np.where(live, t, -1)[..., None]).astype(np.float64)
    return (p - onehot) * np.where(live, np.asarray(dloss, dtype=np.float64), 0.0)[..., None]


def cross_entropy_jvp(logits, targets, tlogits):
    """tloss = sum_v softmax(z)_v tz_v - tz[t]."""
    z = np.asarray(logits, dtype=np.float64)
    tz = np.asarray(tlogits, dtype=np.float64)
    t = np.asarray(targets)
    _, lse = cross_entropy_fwd(z, t)
    live = (t >= 0) & (t < z.shape[-1])
    picked = np.take_along_axis(tz, np.where(live, t, 0)[..., None].astype(np.int64), axis=-1)[..., 0]
    return np.where(live, (np.exp(z - lse[..., None]) * tz).sum(axis=-1) - picked, 0.0)


# ---------------------------------------------------------------------------
# 5. Seeded synthetic inputs for the benchmark configurations
# ---------------------------------------------------------------------------

# ---------------------------------------------------------------------------
# 5. Forward mode (tangents): what `jax.jvp` of the same program computes
#    (reference: enzyme_jvp, src/enzyme_ad/jax/primitives.py:1147-1245).  Pinned by
#    <J v, w> = <v, J^T w> against the reverse-mode functions above and by central
#    finite differences (tests/test_oracle_llama.py).
# ---------------------------------------------------------------------------

def rmsnorm_jvp(x, gamma, tx, tgamma, eps=EPS):
    """ty = gamma (r tx - x r^3 mean(x tx)) + tgamma x r."""
    r = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return gamma * (r * tx - x * r ** 3 * np.mean(x * tx, axis=-1, keepdims=True)) + tgamma * x * r


def linear_jvp(x, w, tx, tw):
    return tx @ w.T + x @ tw.T


def swiglu_jvp(a, b, ta, tb):
    s = 1.0 / (1.0 + np.exp(-a))
    return ta * b * s * (1.0 + a * (1.0 - s)) + tb * a * s


def attention_jvp(q, k, v, tq, tk, tv, scale=None, causal=True):
    """tS = scale (tq k^T + q tk^T); tP = P (tS - rowsum(P tS)); to = tP v + P tv."""
    B, h, S, d = q.shape
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * scale
    if causal:
        mask = np.tril(np.ones((S, k.shape[2]), dtype=bool), k=k.shape[2] - S)
        s = np.where(mask, s, -np.inf)
    p = np.exp(s - np.max(s, axis=-1, keepdims=True))
    p = p / np.sum(p, axis=-1, keepdims=True)
    ts = (np.einsum("bhqd,bhkd->bhqk", tq, k) + np.einsum("bhqd,bhkd->bhqk", q, tk)) * scale
    tp = p * (ts - np.sum(p * ts, axis=-1, keepdims=True))
    return np.einsum("bhqk,bhkd->bhqd", tp, v) + np.einsum("bhqk,bhkd->bhqd", p, tv)


def layer_jvp(x, lw, tx, tlw, n_heads, eps=EPS, theta=ROPE_THETA):
    """Tangent of layer_fwd for tangents tx of x and tlw (same keys) of the weights."""
    B, S, D = x.shape
    d = D // n_heads
    cos, sin = rope_angles(S, d, theta, 0, dtype=x.dtype)
    tr = lambda t: _heads(t, n_heads).transpose(0, 2, 1, 3)
    xb = rmsnorm_fwd(x, lw["rms_att_weight"], eps)
    txb = rmsnorm_jvp(x, lw["rms_att_weight"], tx, tlw["rms_att_weight"], eps)
    q, k, v = (linear_fwd(xb, lw[n]) for n in ("wq", "wk", "wv"))
    tq, tk, tv = (linear_jvp(xb, lw[n], txb, tlw[n]) for n in ("wq", "wk", "wv"))
    qr, kr = rope_fwd(_heads(q, n_heads), cos, sin), rope_fwd(_heads(k, n_heads), cos, sin)
    tqr, tkr = rope_fwd(_heads(tq, n_heads), cos, sin), rope_fwd(_heads(tk, n_heads), cos, sin)     # linear
    o, _ = attention_fwd(qr.transpose(0, 2, 1, 3), kr.transpose(0, 2, 1, 3), tr(v), 1.0 / np.sqrt(d), True)
    to = attention_jvp(qr.transpose(0, 2, 1, 3), kr.transpose(0, 2, 1, 3), tr(v), tqr.transpose(0, 2, 1, 3),
                       tkr.transpose(0, 2, 1, 3), tr(tv), 1.0 / np.sqrt(d), True)
    att, tatt = o.transpose(0, 2, 1, 3).reshape(B, S, D), to.transpose(0, 2, 1, 3).reshape(B, S, D)
    x1 = x + linear_fwd(att, lw["wo"])
    tx1 = tx + linear_jvp(att, lw["wo"], tatt, tlw["wo"])
    xb2 = rmsnorm_fwd(x1, lw["rms_ffn_weight"], eps)
    txb2 = rmsnorm_jvp(x1, lw["rms_ffn_weight"], tx1, tlw["rms_ffn_weight"], eps)
    a1, a3 = linear_fwd(xb2, lw["w1"]), linear_fwd(xb2, lw["w3"])
    ta1, ta3 = linear_jvp(xb2, lw["w1"], txb2, tlw["w1"]), linear_jvp(xb2, lw["w3"], txb2, tlw["w3"])
    g, tg = swiglu_fwd(a1, a3), swiglu_jvp(a1, a3, ta1, ta3)
    y = x1 + linear_fwd(g, lw["w2"])
    ty = tx1 + linear_jvp(g, lw["w2"], tg, tlw["w2"])
    return y, ty


def model_jvp(x, weights, tx, tweights, config, eps=EPS, theta=ROPE_THETA):
    """Tangent of model_fwd (activations in, final RMSNorm out) for tangents of x and of every weight."""
    t = tx
    for i in range(config["n_layers"]):
        x, t = layer_jvp(x, _layer_weights(weights, i), t, _layer_weights(tweights, i), config["n_heads"], eps, theta)
    return (rmsnorm_fwd(x, weights["rms_final_weight"], eps),
            rmsnorm_jvp(x, weights["rms_final_weight"], t, tweights["rms_final_weight"], eps))


def forward_step_vjp(x, config, weights, key_cache, value_cache, dy, eps=EPS, theta=ROPE_THETA):
    """Reverse of `forward_step` (the program `jax.vjp` of test/llama.py:35-238 computes):
    cotangents of x, of every weight and of both caches for the output cotangent dy.
    Built from the batched closed forms on a one-token batch: the token at position pos
    attends to the pos cache rows and to its own row, i.e. non-causal attention of one
    query over pos+1 keys; the appended row's cotangent goes to k / v, the others to the
    cache (Concatenate rule, StableHLOAutoDiffOpInterfaceImpl.cpp:2015-2059).  Returns
    (y, dx, dweights, dkey_cache, dvalue_cache); y must equal forward_step's."""
    n_layers, n_heads, D = config["n_layers"], config["n_heads"], config["dim"]
    d = D // n_heads
    pos = key_cache.shape[1]
    scale = 1.0 / np.sqrt(d)
    cos, sin = rope_angles(1, d, theta, pos, dtype=np.float64)
    hd = lambda t: t.reshape(1, -1, n_heads, d).transpose(0, 2, 1, 3)          # [S, D] -> [1, h, S, d]
    unhd = lambda t: t.transpose(0, 2, 1, 3).reshape(-1, D)                    # back to [S, D]
    saved = []
    x = np.asarray(x, dtype=np.float64).reshape(1, 1, D)
    for i in range(n_layers):
        lw = _layer_weights(weights, i)
        xb = rmsnorm_fwd(x, lw["rms_att_weight"], eps)
        q, k, v = linear_fwd(xb, lw["wq"]), linear_fwd(xb, lw["wk"]), linear_fwd(xb, lw["wv"])
        qr = rope_fwd(_heads(q, n_heads), cos, sin).reshape(1, D)
        kr = rope_fwd(_heads(k, n_heads), cos, sin).reshape(1, D)
        K = np.concatenate([key_cache[i], kr], axis=0)
        V = np.concatenate([value_cache[i], v.reshape(1, D)], axis=0)
        o, _ = attention_fwd(hd(qr), hd(K), hd(V), scale, causal=False)
        att = unhd(o).reshape(1, 1, D)
        x1 = x + linear_fwd(att, lw["wo"])
        xb2 = rmsnorm_fwd(x1, lw["rms_ffn_weight"], eps)
        a1, a3 = linear_fwd(xb2, lw["w1"]), linear_fwd(xb2, lw["w3"])
        g = swiglu_fwd(a1, a3)
        saved.append(dict(x=x, xb=xb, qr=qr, K=K, V=V, att=att, x1=x1, xb2=xb2, a1=a1, a3=a3, g=g))
        x = x1 + linear_fwd(g, lw["w2"])
    y = rmsnorm_fwd(x, weights["rms_final_weight"], eps)

    gw = {k: np.zeros_like(np.asarray(weights[k], dtype=np.float64)) for k in LAYER_KEYS}
    dkc, dvc = np.zeros_like(key_cache, dtype=np.float64), np.zeros_like(value_cache, dtype=np.float64)
    dx, gw["rms_final_weight"] = rmsnorm_bwd(x, weights["rms_final_weight"], np.asarray(dy, dtype=np.float64).reshape(1, 1, D), eps)
    for i in reversed(range(n_layers)):
        lw, c = _layer_weights(weights, i), saved[i]
        dg, gw["w2"][i] = linear_bwd(c["g"], lw["w2"], dx)
        da1, da3 = swiglu_bwd(c["a1"], c["a3"], dg)
        dxa, gw["w1"][i] = linear_bwd(c["xb2"], lw["w1"], da1)
        dxb, gw["w3"][i] = linear_bwd(c["xb2"], lw["w3"], da3)
        dx1n, gw["rms_ffn_weight"][i] = rmsnorm_bwd(c["x1"], lw["rms_ffn_weight"], dxa + dxb, eps)
        dx1 = dx + dx1n
        datt, gw["wo"][i] = linear_bwd(c["att"], lw["wo"], dx1)
        dq, dK, dV = attention_bwd(hd(c["qr"]), hd(c["K"]), hd(c["V"]), hd(datt.reshape(1, D)), scale, causal=False)
        dq, dK, dV = unhd(dq), unhd(dK), unhd(dV)
        dkc[i], dvc[i] = dK[:pos], dV[:pos]
        dqp = rope_bwd(_heads(dq.reshape(1, 1, D), n_heads), cos, sin).reshape(1, 1, D)
        dkp = rope_bwd(_heads(dK[pos:].reshape(1, 1, D), n_heads), cos, sin).reshape(1, 1, D)
        dxq, gw["wq"][i] = linear_bwd(c["xb"], lw["wq"], dqp)
        dxk, gw["wk"][i] = linear_bwd(c["xb"], lw["wk"], dkp)
        dxv, gw["wv"][i] = linear_bwd(c["xb"], lw["wv"], dV[pos:].reshape(1, 1, D))
        dxn, gw["rms_att_weight"][i] = rmsnorm_bwd(c["x"], lw["rms_att_weight"], dxq + dxk + dxv, eps)
        dx = dx1 + dxn
    return y.reshape(D), dx.reshape(D), gw, dkc, dvc


def make_weights(config, seed, std=0.02, dtype=np.float32, embedding=True, norm_gain="normal"):
    """Weights drawn with numpy Generator(PCG64(seed)) in a fixed key order.
    `norm_gain`: "normal" draws the RMSNorm gains N(0, std) like every other
    weight (configuration text), "uniform" draws U(0.5, 1.5)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    L, D, H, V = config["n_layers"], config["dim"], config["hidden_dim"], config["vocab_size"]
    shapes = [("rms_att_weight", (L, D)), ("wq", (L, D, D)), ("wk", (L, D, D)), ("wv", (L, D, D)),
              ("wo", (L, D, D)), ("rms_ffn_weight", (L, D)), ("w1", (L, H, D)), ("w2", (L, D, H)),
              ("w3", (L, H, D)), ("rms_final_weight", (D,)), ("wcls", (V, D))]
    if embedding:
        shapes.append(("token_embedding_table", (V, D)))
    w = {}
    for name, shp in shapes:
        if name.startswith("rms_") and norm_gain == "uniform":
            w[name] = rng.uniform(0.5, 1.5, size=shp).astype(dtype)
        else:
            w[name] = (rng.standard_normal(size=shp) * std).astype(dtype)
    return w
