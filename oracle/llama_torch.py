"""CPU oracle, part 3: an independent PyTorch restatement of test/llama.py's model in batched, causal form.

TEST INFRASTRUCTURE ONLY (imported by tests/ and by bench.py's cpu_baseline leg, never by the product package).

Written against the reference's source (test/llama.py:6-28 rmsnorm / softmax / silu, :127-140 rotation of adjacent
pairs, :144-233 the layer, :235-238 final norm and the commented-out classifier), not against oracle/llama_ref.py:
RoPE goes through complex multiplication, attention through torch's scaled_dot_product_attention, gradients through
torch.autograd.  tests/test_oracle_llama.py requires the numpy oracle to agree with it in float64 (value and every
gradient); bench.py times it in float32 on the host cores as the CPU baseline (the reference's own JAX-CPU path needs
jax and a Bazel-built extension, neither of which exists offline).
"""
import torch


def _norm(t, g, eps=1e-5):
    return g * t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps)


def _rotation(S, d, dtype):
    pos = torch.arange(S, dtype=torch.float64)
    freq = 1.0 / torch.pow(torch.tensor(10000.0, dtype=torch.float64), torch.arange(0, d, 2, dtype=torch.float64) / d)
    ang = pos[:, None] * freq[None]
    rot = torch.polar(torch.ones_like(ang), ang)      # e^{i angle}, complex128
    return rot if dtype == torch.float64 else rot.to(torch.complex64)


def _rope(t, rot):
    B, S, nh, d = t.shape
    tc = torch.view_as_complex(t.reshape(B, S, nh, d // 2, 2).contiguous())
    return torch.view_as_real(tc * rot[None, :, None, :]).reshape(B, S, nh, d)


def layer(x, lw, n_heads, rot=None):
    """One decoder layer over x [B, S, D]; lw holds rms_att_weight, wq, wk, wv, wo, rms_ffn_weight, w1, w2, w3."""
    B, S, D = x.shape
    d = D // n_heads
    if rot is None:
        rot = _rotation(S, d, x.dtype)
    xb = _norm(x, lw["rms_att_weight"])
    q = _rope((xb @ lw["wq"].T).reshape(B, S, n_heads, d), rot).transpose(1, 2)
    k = _rope((xb @ lw["wk"].T).reshape(B, S, n_heads, d), rot).transpose(1, 2)
    v = (xb @ lw["wv"].T).reshape(B, S, n_heads, d).transpose(1, 2)
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    x = x + o.transpose(1, 2).reshape(B, S, D) @ lw["wo"].T
    xb = _norm(x, lw["rms_ffn_weight"])
    return x + (torch.nn.functional.silu(xb @ lw["w1"].T) * (xb @ lw["w3"].T)) @ lw["w2"].T


LAYER_KEYS = ("rms_att_weight", "wq", "wk", "wv", "wo", "rms_ffn_weight", "w1", "w2", "w3")


def model(tokens, w, cfg, logits):
    """tokens [B, S] (integer) -> final-norm output [B, S, D] or logits [B, S, V]; w holds stacked per-layer weights."""
    nh = cfg["n_heads"]
    x = w["token_embedding_table"][tokens]
    rot = _rotation(x.shape[1], cfg["dim"] // nh, x.dtype)
    for i in range(cfg["n_layers"]):
        x = layer(x, {k: w[k][i] for k in LAYER_KEYS}, nh, rot)
    x = _norm(x, w["rms_final_weight"])
    return x @ w["wcls"].T if logits else x
