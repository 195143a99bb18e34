"""The reference's width-16 network assembled only from torch library ops (CPU, fp64), used to pin the
float64 variant of the CPU checker (oracle/width16.py): F.embedding, F.rms_norm, F.linear, torch.max over
masked scores, gather, F.gelu, F.silu, F.cross_entropy.  The graph is the one tests/reference.py:50-81 of
the reference describes (pre-RMSNorm blocks, partial RoPE of one radian per position on the first pair of
every head, causal arg-max attention with a GELU gate, SwiGLU(48), mean cross-entropy); nothing is rounded
and no weight is truncated, exactly like Width16(exact=True)."""
import numpy as np
import torch
from torch.nn import functional as F


def forward_backward(entries, flat, x, y, depth):
    """entries: name -> (offset, shape) in the flat order of model.h:12-37.
    Returns logits [B,T,256], the flat gradient of the mean loss, per-token losses [B,T], all fp64."""
    params = {name: torch.tensor(np.asarray(flat[offset:offset + int(np.prod(shape))], np.float64).reshape(shape),
                                 requires_grad=True) for name, (offset, shape) in entries.items()}
    B, T = x.shape
    tx, ty = torch.tensor(x).long(), torch.tensor(y).long()
    positions = torch.arange(T, dtype=torch.float64)
    cos, sin = torch.cos(positions), torch.sin(positions)

    def rope(t):  # t: [B, heads, T, 4]
        x0, x1 = t[..., 0], t[..., 1]
        return torch.stack((x0 * cos - x1 * sin, x0 * sin + x1 * cos, t[..., 2], t[..., 3]), -1)

    h = F.embedding(tx, params["embedding"])
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    for l in range(depth):
        s = f"{l}."
        packed = F.linear(F.rms_norm(h, (16,), params[s + "attention_norm"], eps=1e-6), params[s + "qkv"])
        query, key, value = [a.reshape(B, T, 4, 4).transpose(1, 2) for a in packed.split(16, -1)]
        query, key = rope(query), rope(key)
        scores = query @ key.transpose(-1, -2)
        top, index = scores.masked_fill(~mask, -1e30).max(-1, keepdim=True)
        selected = value.gather(2, index.expand(-1, -1, -1, 4))
        a = (selected * F.gelu(top)).transpose(1, 2).reshape(B, T, 16)
        h = h + F.linear(a, params[s + "attention"])
        gate, up = F.linear(F.rms_norm(h, (16,), params[s + "mlp_norm"], eps=1e-6),
                            torch.cat((params[s + "gate"], params[s + "up"]))).split(48, -1)
        h = h + F.linear(F.silu(gate) * up, params[s + "down"])
    logits = F.linear(F.rms_norm(h, (16,), params["final_norm"], eps=1e-6), params["head"])
    loss = F.cross_entropy(logits.flatten(0, 1), ty.flatten(), reduction="none").reshape(B, T)
    loss.mean().backward()
    grad = np.zeros(len(flat), np.float64)
    for name, (offset, shape) in entries.items():
        grad[offset:offset + int(np.prod(shape))] = params[name].grad.numpy().ravel()
    return logits.detach().numpy(), grad, loss.detach().numpy()
