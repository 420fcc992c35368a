"""Writes encoder_layer_c1.npz with torch.nn.TransformerEncoderLayer (an independent library
implementation of the post-LN encoder layer) on the seeded dense BERT-base configuration."""
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

H, NH, FF, S = 768, 12, 3072, 128


def seeded_params(seed=1):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g) * 0.02
    return {"Wqkv": rn(3 * H, H), "Wo": rn(H, H), "W1": rn(FF, H), "W2": rn(H, FF),
            "x": torch.randn(S, H, generator=g)}


def main():
    p = seeded_params()
    layer = torch.nn.TransformerEncoderLayer(H, NH, FF, dropout=0.0, activation=lambda t: F.gelu(t, approximate="tanh"),
                                             layer_norm_eps=1e-5, batch_first=True, norm_first=False)
    with torch.no_grad():
        layer.self_attn.in_proj_weight.copy_(p["Wqkv"]); layer.self_attn.in_proj_bias.zero_()
        layer.self_attn.out_proj.weight.copy_(p["Wo"]); layer.self_attn.out_proj.bias.zero_()
        layer.linear1.weight.copy_(p["W1"]); layer.linear1.bias.zero_()
        layer.linear2.weight.copy_(p["W2"]); layer.linear2.bias.zero_()
        for ln in (layer.norm1, layer.norm2):
            ln.weight.fill_(1.0); ln.bias.zero_()
        layer.eval()
        y = layer(p["x"][None])[0]
    np.savez(Path(__file__).with_name("encoder_layer_c1.npz"), y_head=y[:8].numpy(),
             y_sum=np.float64(y.double().sum().item()), y_abs_sum=np.float64(y.double().abs().sum().item()))


if __name__ == "__main__":
    main()
