"""Independent fp64 torch.autograd statement of the LLaMA step (test helper).

Written from the model definition (RMSNorm, rotate-half RoPE, causal softmax
attention, SwiGLU, softmax cross-entropy), not from the oracle's code, so that
it pins the oracle's composed gradients.  src/librarium/llama.rs:420-548.
"""
import numpy as np
import torch


def make_inputs(cfg_dict, seed=0, std=0.02, norm_mean=0.0, grad_scale=1.0):
    """Seeded synthetic parameters / tokens for a config (flat f16 block + inputs).

    Matrices and the embedding ~N(0, std); norm weights ~N(norm_mean, std).
    Labels are the ids shifted by one; loss scale = grad_scale / (S - 1) with
    position 0 zeroed (examples/open_llama_3b_train.rs:521-530)."""
    from oracle import oracle as o
    cfg = o.Cfg(**cfg_dict)
    r = np.random.default_rng(seed)
    parts = []
    for name, shp in o.param_layout(cfg):
        mean = norm_mean if name.endswith("norm") else 0.0
        parts.append((mean + r.standard_normal(shp) * std).astype(np.float16).ravel())
    flat = np.concatenate(parts)
    tok = r.integers(0, cfg.V, cfg.S).astype(np.uint16)
    lm_tok = np.concatenate([tok[1:], tok[:1]]).astype(np.uint16)
    scale = np.full(cfg.S, grad_scale / (cfg.S - 1), np.float32)
    scale[0] = 0.0
    return cfg, flat, tok, lm_tok, scale


def torch_step(cfg, params, tok, lm_tok, scale):
    """params: dict name -> np.float16 array.  Returns (loss [S], grads dict) in fp64."""
    S, D, H, Dh, F, V, L = cfg.S, cfg.D, cfg.H, cfg.Dh, cfg.F, cfg.V, cfg.L
    P = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in params.items()}
    tok_t = torch.tensor(tok.astype(np.int64))
    tgt = torch.tensor(lm_tok.astype(np.int64))
    i = torch.arange(Dh // 2, dtype=torch.float64)
    inv = 10000.0 ** (-2.0 * i / Dh)
    fr = torch.arange(S, dtype=torch.float64)[:, None] * inv[None, :]
    fr = torch.cat([fr, fr], 1)
    cos, sin = fr.cos()[:, None, :], fr.sin()[:, None, :]

    def norm(x, w):
        return w * x / torch.sqrt((x * x).mean(1, keepdim=True) + cfg.eps)

    def rope(x):
        x = x.view(S, H, Dh)
        rot = torch.cat([-x[..., Dh // 2:], x[..., :Dh // 2]], -1)
        return x * cos + rot * sin

    x = P["embed"][tok_t]
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1)
    for l in range(L):
        g = lambda n: P["l%d.%s" % (l, n)]
        hN = norm(x, g("pre_norm"))
        q, k = rope(hN @ g("q").T), rope(hN @ g("k").T)
        v = (hN @ g("v").T).view(S, H, Dh)
        sc = torch.einsum("ihd,jhd->hij", q, k) / np.sqrt(Dh)
        sc = sc.masked_fill(mask[None], float("-inf"))
        a = torch.einsum("hij,jhd->ihd", torch.softmax(sc, -1), v).reshape(S, D)
        x = x + a @ g("o").T
        hN = norm(x, g("post_norm"))
        x = x + (torch.nn.functional.silu(hN @ g("gate").T) * (hN @ g("up").T)) @ g("down").T
    logit = norm(x, P["head_norm"]) @ P["lm_head"].T
    loss = torch.nn.functional.cross_entropy(logit, tgt, reduction="none")
    (loss * torch.tensor(scale.astype(np.float64))).sum().backward()
    return loss.detach().numpy(), {k: v.grad.numpy() for k, v in P.items()}, logit.detach().numpy()
