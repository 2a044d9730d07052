"""The llama2-style transformer of the reference's test/llama.py, batched and
causal, written with the HIP operators of `enzyme_ad.jax.ops`.

`forward(x, config, weights, ...)` keeps the reference's argument order
(test/llama.py:35) where that makes sense: activations [B, S, dim] replace the
single-token vector, the causal mask replaces the KV cache (a token at
position t attends to rows 0..t, exactly what the step form sees in its
cache).  Weight names and layouts are the reference's: matrices are [out, in]
and applied as `w @ x` (:149).
"""
from . import ops

LAYER_KEYS = ("rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3")


def layer(x, lw, n_heads, eps=1e-5, theta=10000.0):
    """One decoder layer (test/llama.py:144-233).  x: [B, S, dim]."""
    xb = ops.rmsnorm(x, lw["rms_att_weight"], eps)                 # :145
    att = ops.attention_block(xb, lw["wq"], lw["wk"], lw["wv"], n_heads, theta)     # :149-209 (RoPE in the epilogues)
    x = ops.matmul_nt(att, lw["wo"], residual=x)                   # :211-215
    xb = ops.rmsnorm(x, lw["rms_ffn_weight"], eps)                 # :219
    return ops.ffn(xb, lw["w1"], lw["w3"], lw["w2"], residual=x)   # :224-233 (SwiGLU in the GEMM epilogues)


def forward(x, config, weights, logits=False, eps=1e-5, theta=10000.0):
    """Whole model.  x: activations [B, S, dim], or int32 tokens [B, S] when
    `weights` holds `token_embedding_table` (the lookup commented out at
    test/llama.py:109-113).  Returns the final RMSNorm of the residual stream
    (:235) or, with `logits`, its `wcls` projection (:236)."""
    n_layers, n_heads = config["n_layers"], config["n_heads"]
    if not x.is_floating_point():
        x = ops.embedding(x, weights["token_embedding_table"])
    for i in range(n_layers):
        lw = {k: ops.select(weights[k], i) for k in LAYER_KEYS}
        x = layer(x, lw, n_heads, eps, theta)
    x = ops.rmsnorm(x, weights["rms_final_weight"], eps)
    if logits:
        x = ops.matmul_nt(x, weights["wcls"])
    return x


def loss(x, targets, config, weights, eps=1e-5, theta=10000.0):
    """Mean over all tokens of the softmax cross-entropy of `forward(..., logits=True)` against int32 `targets`
    `[B, S]`: a scalar fp32 tensor.  What a training step differentiates once the classifier commented out at
    test/llama.py:236 is switched on."""
    import torch

    from . import hlo_ops as H

    per_token = ops.cross_entropy(forward(x, config, weights, logits=True, eps=eps, theta=theta), targets)
    total = H.reduce("add", per_token, range(per_token.dim()))
    return H.binary("multiply", total, torch.full((), 1.0 / targets.numel(), dtype=torch.float32, device=total.device))


def forward_step(x, config, weights, key_cache, value_cache, eps=1e-5, theta=10000.0):
    """The reference's own single-token form, argument for argument
    (test/llama.py:35-238): x is the residual stream of one token [dim];
    key_cache / value_cache are [n_layers, pos, kv_dim] and the token sits at
    position pos = key_cache.shape[1].  Returns the final RMSNorm of the residual
    stream.  Every projection is a mat-vec (weight-bandwidth-bound kernels)."""
    n_layers, n_heads = config["n_layers"], config["n_heads"]
    if config.get("n_kv_heads", n_heads) != n_heads:
        # the reference reshapes k with `dim`, not `kv_dim` (:162,171): it only runs with equal head counts
        raise ValueError("forward_step: n_kv_heads must equal n_heads")
    dim = x.shape[-1]
    pos = key_cache.shape[1]
    for i in range(n_layers):
        lw = {k: ops.select(weights[k], i) for k in LAYER_KEYS}
        xb = ops.rmsnorm(x, lw["rms_att_weight"], eps)                                    # :145
        q = ops.matmul_nt(xb, lw["wq"])                                                   # :149-157
        k = ops.matmul_nt(xb, lw["wk"])
        v = ops.matmul_nt(xb, lw["wv"])
        q = ops.reshape(ops.rope(ops.reshape(q, (1, 1, dim)), n_heads, theta, pos0=pos), (dim,))   # :161-168
        k = ops.reshape(ops.rope(ops.reshape(k, (1, 1, dim)), n_heads, theta, pos0=pos), (dim,))
        key_cache_l = ops.append_row(ops.select(key_cache, i), k)                         # :170-175
        value_cache_l = ops.append_row(ops.select(value_cache, i), v)
        att = ops.attention_step(q, key_cache_l, value_cache_l, n_heads)                  # :178-209
        x = ops.matmul_nt(att, lw["wo"], residual=x)                                      # :211-215
        xb = ops.rmsnorm(x, lw["rms_ffn_weight"], eps)                                    # :219
        h1 = ops.matmul_nt(xb, lw["w1"])                                                  # :224-225
        h3 = ops.matmul_nt(xb, lw["w3"])
        g = ops.swiglu(h1, h3)                                                            # :227-229
        x = ops.matmul_nt(g, lw["w2"], residual=x)                                        # :231-233
    return ops.rmsnorm(x, weights["rms_final_weight"], eps)                               # :235
