"""A GPT built only from torch library ops (CPU, fp64), used to pin the CPU checker's model.
Structure follows tests/reference.py:50-81 of the reference (pre-norm blocks, truncated bf16
compute weights with straight-through gradients, mean cross-entropy), with the operators the
target names: LayerNorm, softmax attention, GELU MLP, learned positions."""
import numpy as np
import torch
from torch.nn import functional as F


class Truncate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        bits = x.detach().float().contiguous().view(torch.int32) & -65536
        return bits.view(torch.float32).double()

    @staticmethod
    def backward(ctx, grad):
        return grad


def forward_backward(layout, flat, x, y, heads, eps=1e-5):
    """Returns logits [B,T,V], flat gradient, per-token loss [B,T] in fp64."""
    params = {}
    for name, offset, shape in layout.entries:
        params[name] = torch.tensor(flat[offset:offset + int(np.prod(shape))].reshape(shape),
                                    dtype=torch.float64, requires_grad=True)

    def weight(name):
        return Truncate.apply(params[name])

    B, T = x.shape
    tx, ty = torch.tensor(x).long(), torch.tensor(y).long()
    h = F.embedding(tx, weight("embedding")) + weight("positions")[None, :T]
    d = h.shape[-1]
    depth = sum(1 for n, _, _ in layout.entries if n.endswith(".qkv"))
    for l in range(depth):
        s = f"{l}."
        n1 = F.layer_norm(h, (d,), params[s + "ln1_g"], params[s + "ln1_b"], eps)
        q, k, v = [t.reshape(B, T, heads, d // heads).transpose(1, 2)
                   for t in F.linear(n1, weight(s + "qkv")).split(d, -1)]
        o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        h = h + F.linear(o.transpose(1, 2).reshape(B, T, d), weight(s + "attn_out"))
        n2 = F.layer_norm(h, (d,), params[s + "ln2_g"], params[s + "ln2_b"], eps)
        h = h + F.linear(F.gelu(F.linear(n2, weight(s + "mlp_up"))), weight(s + "mlp_down"))
    logits = F.linear(F.layer_norm(h, (d,), params["lnf_g"], params["lnf_b"], eps), weight("head"))
    loss = F.cross_entropy(logits.flatten(0, 1), ty.flatten(), reduction="none").reshape(B, T)
    loss.mean().backward()
    grad = np.concatenate([params[name].grad.numpy().ravel() for name, _, _ in layout.entries])
    return logits.detach().numpy(), grad, loss.detach().numpy()
