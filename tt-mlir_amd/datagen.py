"""Seeded synthetic inputs of the benchmark configurations.

One generator feeds both the CPU checker and the GPU run, so inputs are identical.  Like the
reference builder (tools/builder/base/builder.py:119, 659-679) tensors come from torch.randn
under torch.manual_seed(seed), always generated on the CPU.
"""
import torch


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def randn(shape, seed=0, std=1.0, dtype=torch.float32):
    x = torch.randn(shape, generator=_gen(seed), dtype=torch.float32)
    if std != 1.0:
        x = x * std
    return x.to(dtype)


def c1_matmul(seed=0):
    """Config 1: bf16 matmul [256,512] x [512,256], N(0,1)."""
    g = _gen(seed)
    a = torch.randn((256, 512), generator=g).to(torch.bfloat16)
    b = torch.randn((512, 256), generator=g).to(torch.bfloat16)
    return a, b


def c2_outliers(rows=8192, cols=8192, seed=0, frac=0.01, scale=100.0):
    """Config 2: fp32 N(0,1) with a seeded Bernoulli(frac) mask of entries scaled by `scale`."""
    g = _gen(seed)
    x = torch.randn((rows, cols), generator=g)
    mask = torch.rand((rows, cols), generator=g) < frac
    x[mask] *= scale
    return x


def c3_linear(M, K=4096, N=14336, seed=0):
    """Config 3: bf16 activations [M,K] N(0,1); weights [K,N] N(0,0.02) (to be packed bfp8_b);
    bias [N] N(0,0.02) bf16."""
    g = _gen(seed)
    a = torch.randn((M, K), generator=g).to(torch.bfloat16)
    w = torch.randn((K, N), generator=g) * 0.02
    bias = (torch.randn((N,), generator=g) * 0.02).to(torch.bfloat16)
    return a, w, bias


def c4_mlp(tokens=512, hidden=4096, ffn=14336, seed=0):
    """Config 4: Llama-style MLP block inputs and weights."""
    g = _gen(seed)
    x = torch.randn((tokens, hidden), generator=g).to(torch.bfloat16)
    norm_w = (1.0 + 0.02 * torch.randn((hidden,), generator=g)).to(torch.bfloat16)
    wg = torch.randn((hidden, ffn), generator=g) * 0.02
    wu = torch.randn((hidden, ffn), generator=g) * 0.02
    wd = torch.randn((ffn, hidden), generator=g) * 0.02
    return dict(x=x, norm_w=norm_w, wg=wg, wu=wu, wd=wd, eps=1e-5)


def c5_decoder(seq=2048, hidden=4096, n_q=32, n_kv=8, head_dim=128, ffn=14336, seed=0):
    """Config 5: Llama-3-8B-shaped decoder layer, batch 1."""
    g = _gen(seed)
    d = dict(seq=seq, hidden=hidden, n_q=n_q, n_kv=n_kv, head_dim=head_dim, ffn=ffn, eps=1e-5)
    d["x"] = torch.randn((1, seq, hidden), generator=g).to(torch.bfloat16)
    d["attn_norm_w"] = (1.0 + 0.02 * torch.randn((hidden,), generator=g)).to(torch.bfloat16)
    d["wq"] = torch.randn((hidden, n_q * head_dim), generator=g) * 0.02
    d["wk"] = torch.randn((hidden, n_kv * head_dim), generator=g) * 0.02
    d["wv"] = torch.randn((hidden, n_kv * head_dim), generator=g) * 0.02
    d["wo"] = torch.randn((n_q * head_dim, hidden), generator=g) * 0.02
    d["mlp_norm_w"] = (1.0 + 0.02 * torch.randn((hidden,), generator=g)).to(torch.bfloat16)
    d["wg"] = torch.randn((hidden, ffn), generator=g) * 0.02
    d["wu"] = torch.randn((hidden, ffn), generator=g) * 0.02
    d["wd"] = torch.randn((ffn, hidden), generator=g) * 0.02
    return d
