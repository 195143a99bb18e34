"""CPU checker for the reference's own width-16 network (numpy).

TEST INFRASTRUCTURE ONLY: imported by tests/ alone; the shipped package never imports it.

Restates, with every bf16 rounding point, the model the reference trains behind the plain ``Config``:
width 16, 4 heads of 4, vocabulary 256, RMSNorm(eps 1e-6), partial RoPE (first pair of each head,
one radian per position), causal arg-max attention with a GELU gate, SwiGLU(48), tied nothing.
  forward  : cuda/model.cuh:8-58, tests/reference.py:50-81
  backward : cuda/model.cuh:59-99, cuda/ops.cuh:57-144, cuda/attention.cuh:72-106
  layout   : model.h:12-37
  optimizer: cuda/optim.cuh:5-119 (mantissa-preserving AdamW for embedding / head / scales, Muon with
             a bf16 Newton-Schulz iteration for the hidden matrices)
``exact=True`` runs the same graph in float64 without any rounding or weight truncation; that variant
is what finite differences pin, and the rounded variant is checked against it.

What pins it (tests/test_oracle_width16.py): the float64 variant against the same network assembled only from
torch library ops and autograd (tests/torch_width16.py: logits 1e-9, every gradient tensor 1e-6); finite
differences of the float64 variant for every parameter tensor; rounded against float64 within bf16 resolution; the RoPE table against
float32(cos k), float32(sin k) and the eight constants of cuda/attention.cuh:7-14; the tie rule
(first key wins); causality; the AdamW part against torch.optim.AdamW and the Muon part against
torch.optim.Muon (library routines); the 64-small-steps known answer of tests/verify.py:108-127.
"""
import math

import numpy as np

WIDTH, HEADS, HEAD_DIM, VOCAB, FFN = 16, 4, 4, 256, 48


def layout(depth):
    """name -> (offset, shape), in the flat order of model.h:12-37."""
    entries, n = {}, 0

    def take(name, shape):
        nonlocal n
        entries[name] = (n, shape)
        n += int(np.prod(shape))

    take("embedding", (VOCAB, WIDTH))
    for l in range(depth):
        take(f"{l}.attention_norm", (WIDTH,))
        take(f"{l}.qkv", (3 * WIDTH, WIDTH))
        take(f"{l}.attention", (WIDTH, WIDTH))
        take(f"{l}.mlp_norm", (WIDTH,))
        take(f"{l}.gate", (FFN, WIDTH))
        take(f"{l}.up", (FFN, WIDTH))
        take(f"{l}.down", (WIDTH, FFN))
    take("final_norm", (WIDTH,))
    take("head", (VOCAB, WIDTH))
    return entries, n


def parameter_count(depth):
    return layout(depth)[1]


def is_scale(name):
    return name.endswith("norm")


def is_hidden_matrix(name):
    return name.rsplit(".", 1)[-1] in ("qkv", "attention", "gate", "up", "down")


def rn(x):
    """float32 -> nearest-even bf16, returned as float32."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + (((b >> 16) & 1) + 0x7FFF)) & np.uint32(0xFFFF0000)).view(np.float32)


def truncate(x):
    """The bf16 compute weight: high half of the fp32 master (cuda/ops.cuh:6-14)."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)


def rope_table(context):
    """float32(cos k), float32(sin k): cuda/attention.cuh:7-14, tests/reference.py:57-58."""
    k = np.arange(context, dtype=np.float64)
    return np.cos(k).astype(np.float32), np.sin(k).astype(np.float32)


_erf = np.vectorize(math.erf, otypes=[np.float64])


class Width16:
    def __init__(self, depth, context, batch, exact=False):
        self.depth, self.context, self.sequences, self.exact = depth, context, batch, exact
        self.entries, self.count = layout(depth)
        self.real = np.float64 if exact else np.float32

    # -- helpers ---------------------------------------------------------------------------------
    def r(self, x):
        return np.asarray(x, dtype=np.float64) if self.exact else rn(np.asarray(x, dtype=np.float32))

    def split(self, flat):
        flat = np.asarray(flat)
        out = {}
        for name, (offset, shape) in self.entries.items():
            w = flat[offset:offset + int(np.prod(shape))].reshape(shape)
            if self.exact:
                out[name] = w.astype(np.float64)
            else:
                out[name] = w.astype(np.float32) if is_scale(name) else truncate(w.astype(np.float32))
        return out

    def linear(self, x, w):
        """bf16 x bf16 products, wide accumulation, one rounding (cuda/mma.cuh:77-108)."""
        return self.r(x.astype(np.float64) @ w.astype(np.float64).T)

    def norm(self, x, scale):
        v = x.astype(self.real)
        inv = 1.0 / np.sqrt((v * v).sum(-1, keepdims=True) / WIDTH + self.real(1e-6))
        return self.r(v * inv * scale), inv

    def rope(self, qkv, inverse=False):
        """rotate the first pair of every query and key head, unfused products (cuda/attention.cuh:19-30)"""
        cos, sin = rope_table(self.context)
        if self.exact:
            k = np.arange(self.context, dtype=np.float64)
            cos, sin = np.cos(k), np.sin(k)
        if inverse:
            sin = -sin
        out = qkv.copy()
        cos, sin = cos[None, :, None], sin[None, :, None]
        for base in (0, WIDTH):
            x = qkv[..., base:base + WIDTH:HEAD_DIM].astype(self.real)
            y = qkv[..., base + 1:base + WIDTH:HEAD_DIM].astype(self.real)
            out[..., base:base + WIDTH:HEAD_DIM] = self.r(self.real(1) * (x * cos) - (y * sin))
            out[..., base + 1:base + WIDTH:HEAD_DIM] = self.r(self.real(1) * (x * sin) + (y * cos))
        return out

    # -- forward -----------------------------------------------------------------------------------
    def forward(self, flat, x, keep=False):
        """x: [batch, context] uint8 -> logits [batch, context, 256] (float32 values of bf16 logits)."""
        p = self.split(flat)
        B, T = x.shape
        h = p["embedding"][x.astype(np.int64)]
        saved = []
        for l in range(self.depth):
            s = {"x": h}
            n1, _ = self.norm(h, p[f"{l}.attention_norm"])
            qkv = self.rope(self.linear(n1, p[f"{l}.qkv"]))
            q = qkv[..., :WIDTH].reshape(B, T, HEADS, HEAD_DIM).astype(self.real)
            k = qkv[..., WIDTH:2 * WIDTH].reshape(B, T, HEADS, HEAD_DIM).astype(self.real)
            v = qkv[..., 2 * WIDTH:].reshape(B, T, HEADS, HEAD_DIM)
            # scores[b, head, query, key], accumulated in the compute type in key order c = 0..3
            scores = np.zeros((B, HEADS, T, T), dtype=self.real)
            for c in range(HEAD_DIM):
                scores += q[:, :, :, c].transpose(0, 2, 1)[:, :, :, None] * k[:, :, :, c].transpose(0, 2, 1)[:, :, None, :]
            mask = np.tril(np.ones((T, T), dtype=bool))
            scores = np.where(mask, scores, -np.inf)
            selected = scores.argmax(-1)  # first index wins ties (cuda/attention.cuh:41-44)
            top = np.take_along_axis(scores, selected[..., None], -1)[..., 0]  # [B, heads, T]
            e = 1.0 + _erf(top.astype(np.float64) * 0.7071067811865475).astype(self.real)
            gate = (self.real(0.5) * top * e).astype(self.real)
            deriv = (self.real(0.5) * e + top * self.real(0.3989422804014327) * np.exp(self.real(-0.5) * top * top)).astype(self.real)
            vh = v.transpose(0, 2, 1, 3)  # [B, heads, T, 4]
            chosen = np.take_along_axis(vh, selected[..., None].repeat(HEAD_DIM, -1), 2)
            a = self.r(chosen.astype(self.real) * gate[..., None]).transpose(0, 2, 1, 3).reshape(B, T, WIDTH)
            middle = self.r(self.linear(a, p[f"{l}.attention"]).astype(self.real) + h.astype(self.real))
            n2, _ = self.norm(middle, p[f"{l}.mlp_norm"])
            gu = self.linear(n2, np.concatenate([p[f"{l}.gate"], p[f"{l}.up"]]))
            g, u = gu[..., :FFN].astype(self.real), gu[..., FFN:].astype(self.real)
            sig = 1.0 / (1.0 + np.exp(-g))
            activated = self.r(g * sig)
            act = self.r(activated.astype(self.real) * u)
            h = self.r(self.linear(act, p[f"{l}.down"]).astype(self.real) + middle.astype(self.real))
            s.update(qkv=qkv, selected=selected, gate=gate, deriv=deriv, a=a, middle=middle, n1=n1, n2=n2,
                     gu=gu, sig=sig, activated=activated, act=act)
            saved.append(s)
        nf, _ = self.norm(h, p["final_norm"])
        logits = self.linear(nf, p["head"])
        if keep:
            return logits, (p, saved, h, nf)
        return logits

    @staticmethod
    def token_losses(logits, y):
        z = logits.astype(np.float64)
        high = z.max(-1, keepdims=True)
        lse = high[..., 0] + np.log(np.exp(z - high).sum(-1))
        return lse - np.take_along_axis(z, y.astype(np.int64)[..., None], -1)[..., 0]

    # -- backward --------------------------------------------------------------------------------
    def norm_backward(self, x, dy, scale, grads, name):
        v, g = x.astype(self.real), dy.astype(self.real)
        inv = 1.0 / np.sqrt((v * v).sum(-1, keepdims=True) / WIDTH + self.real(1e-6))
        z = v * inv
        dz = g * scale
        value = (dz - z * (dz * z).sum(-1, keepdims=True) / WIDTH) * inv
        grads[name] = (g * z).astype(np.float64).reshape(-1, WIDTH).sum(0)
        return self.r(value)

    def linear_backward(self, x, dy, w, grads, name):
        X = x.reshape(-1, x.shape[-1]).astype(np.float64)
        D = dy.reshape(-1, dy.shape[-1]).astype(np.float64)
        grads[name] = D.T @ X
        return self.r(dy.astype(np.float64) @ w.astype(np.float64))

    def batch(self, flat, x, y):
        """-> logits [B,T,256] float32, flat gradient of the mean loss (float32), per-position mean losses."""
        B, T = x.shape
        logits, (p, saved, h, nf) = self.forward(flat, x, keep=True)
        losses = self.token_losses(logits, y)
        z = logits.astype(np.float64)
        prob = np.exp(z - z.max(-1, keepdims=True))
        prob /= prob.sum(-1, keepdims=True)
        onehot = np.zeros_like(prob)
        np.put_along_axis(onehot, y.astype(np.int64)[..., None], 1.0, -1)
        dlogits = self.r(((prob - onehot) / (B * T)).astype(self.real))
        g = {}
        dn = self.linear_backward(nf, dlogits, p["head"], g, "head")
        dh = self.norm_backward(h, dn, p["final_norm"], g, "final_norm")
        for l in reversed(range(self.depth)):
            s = saved[l]
            dact = self.linear_backward(s["act"], dh, p[f"{l}.down"], g, f"{l}.down")
            gate_in, u = s["gu"][..., :FFN].astype(self.real), s["gu"][..., FFN:].astype(self.real)
            dy = dact.astype(self.real)
            da = self.r(dy * u)
            sig = s["sig"]
            dgate = self.r(da.astype(self.real) * sig * (1.0 + gate_in * (1.0 - sig)))
            dup = self.r(dy * s["activated"].astype(self.real))
            dgu = np.concatenate([dgate, dup], -1)
            w_gu = np.concatenate([p[f"{l}.gate"], p[f"{l}.up"]])
            packed = {}
            dn2 = self.linear_backward(s["n2"], dgu, w_gu, packed, "gu")
            g[f"{l}.gate"], g[f"{l}.up"] = packed["gu"][:FFN], packed["gu"][FFN:]
            dh = self.r(dh.astype(self.real) + self.norm_backward(s["middle"], dn2, p[f"{l}.mlp_norm"], g, f"{l}.mlp_norm").astype(self.real))
            dattn = self.linear_backward(s["a"], dh, p[f"{l}.attention"], g, f"{l}.attention")
            # arg-max attention backward (cuda/attention.cuh:72-106)
            qkv, selected = s["qkv"], s["selected"]
            q = qkv[..., :WIDTH].reshape(B, T, HEADS, HEAD_DIM).transpose(0, 2, 1, 3).astype(self.real)
            k = qkv[..., WIDTH:2 * WIDTH].reshape(B, T, HEADS, HEAD_DIM).transpose(0, 2, 1, 3).astype(self.real)
            v = qkv[..., 2 * WIDTH:].reshape(B, T, HEADS, HEAD_DIM).transpose(0, 2, 1, 3).astype(self.real)
            dyh = dattn.reshape(B, T, HEADS, HEAD_DIM).transpose(0, 2, 1, 3).astype(self.real)
            index = selected[..., None].repeat(HEAD_DIM, -1)
            dt = np.zeros(selected.shape, dtype=self.real)
            chosen_v = np.take_along_axis(v, index, 2)
            for c in range(HEAD_DIM):
                dt += dyh[..., c] * chosen_v[..., c]
            dt = dt * s["deriv"]
            dq = dt[..., None] * np.take_along_axis(k, index, 2)
            dk = np.zeros_like(k)
            dv = np.zeros_like(v)
            for query in range(T):  # keys accumulate their queries in query order
                key = selected[:, :, query]
                bi, hi = np.meshgrid(np.arange(B), np.arange(HEADS), indexing="ij")
                dk[bi, hi, key] += dt[:, :, query, None] * q[:, :, query]
                dv[bi, hi, key] += dyh[:, :, query] * s["gate"][:, :, query, None]
            dqkv = np.concatenate([t.transpose(0, 2, 1, 3).reshape(B, T, WIDTH) for t in (dq, dk, dv)], -1)
            dqkv = self.rope(self.r(dqkv), inverse=True)
            dn1 = self.linear_backward(s["n1"], dqkv, p[f"{l}.qkv"], g, f"{l}.qkv")
            dh = self.r(dh.astype(self.real) + self.norm_backward(s["x"], dn1, p[f"{l}.attention_norm"], g, f"{l}.attention_norm").astype(self.real))
        emb = np.zeros((VOCAB, WIDTH))
        np.add.at(emb, x.astype(np.int64).reshape(-1), dh.reshape(-1, WIDTH).astype(np.float64))
        g["embedding"] = emb
        out = np.zeros(self.count, dtype=np.float64)
        for name, (offset, shape) in self.entries.items():
            out[offset:offset + int(np.prod(shape))] = g[name].reshape(-1)
        position_losses = losses.mean(0)
        if self.exact:
            return logits, out, position_losses
        return logits.astype(np.float32), out.astype(np.float32), position_losses.astype(np.float32)

    def mean_loss(self, flat, x, y):
        return float(self.token_losses(self.forward(flat, x), y).mean())


# -- optimizer (cuda/optim.cuh) ----------------------------------------------------------------------
def newton_schulz(u, steps):
    """cuda/optim.cuh:17-62 on one matrix: bf16 storage, fp32-wide products, quintic 3.4445 / -4.775 / 2.0315.
    u: rows x cols float32 update; returns the orthogonalised update in the same orientation."""
    rows, cols = u.shape
    wide = rn(u).T.copy() if rows > cols else rn(u).copy()  # 16 x n
    scalar = lambda value: float(rn(np.array([value], np.float32))[0])
    norm = max(scalar(math.sqrt(float((wide.astype(np.float64) ** 2).sum()))), scalar(1e-7))
    wide = rn(wide / np.float32(norm))
    for _ in range(steps):
        a = rn((wide.astype(np.float64) @ wide.astype(np.float64).T).astype(np.float32))
        a2 = (a.astype(np.float64) @ a.astype(np.float64)).astype(np.float32)
        work = rn(np.float32(-4.775) * a + np.float32(2.0315) * a2)
        product = (work.astype(np.float64) @ wide.astype(np.float64)).astype(np.float32)
        wide = rn(np.float32(3.4445) * wide + product)
    return wide.T if rows > cols else wide


class Optimizer:
    """State and one update of the reference's optimizer pair on a flat fp32 parameter vector."""

    def __init__(self, depth, learning_rate=0.0006, muon_lr=0.02, beta1=0.9, beta2=0.95, momentum=0.95,
                 weight_decay=0.1, epsilon=1e-8, clip=1.0, ns_steps=5):
        self.entries, self.count = layout(depth)
        self.lr, self.muon_lr, self.beta1, self.beta2, self.mu = learning_rate, muon_lr, beta1, beta2, momentum
        self.wd, self.eps, self.clip, self.ns_steps = weight_decay, epsilon, clip, ns_steps
        self.m = np.zeros(self.count, np.float32)
        self.v = np.zeros(self.count, np.float32)
        self.step = 0

    def update(self, w, grad, rates=None):
        """w, grad float32 flat; rates = (multiplier, momentum) of the OneCycle point or None.  Returns new w."""
        f = np.float32
        w, grad = w.astype(np.float32).copy(), grad.astype(np.float32)
        norm = np.float32(np.sqrt(np.float32((grad.astype(np.float64) ** 2).sum())))
        clip = f(min(1.0, self.clip / (float(norm) + 1e-6))) if self.clip > 0 else f(1)
        multiplier, beta1, mu = f(1), f(self.beta1), f(self.mu)
        if rates is not None:
            multiplier, beta1, mu = f(rates[0]), f(rates[1]), f(rates[1])
        lr = f(self.lr) * multiplier
        bc1 = f(1) - f(math.pow(float(beta1), self.step + 1))
        bc2 = f(1) - f(math.pow(float(f(self.beta2)), self.step + 1))
        for name, (offset, shape) in self.entries.items():
            sl = slice(offset, offset + int(np.prod(shape)))
            g = grad[sl] * clip
            if is_hidden_matrix(name):
                m = self.m[sl] + (f(1) - mu) * (g - self.m[sl])
                self.m[sl] = m
                u = g + mu * (m - g)
                rows, cols = shape
                o = newton_schulz(u.reshape(shape), self.ns_steps).reshape(-1)
                mlr = f(self.muon_lr) * multiplier
                adjusted = mlr * f(math.sqrt(max(1.0, rows / cols)))
                w[sl] = w[sl] * (f(1) - mlr * f(self.wd)) - adjusted * o
            else:
                decay = f(self.wd) if name == "head" else f(0)
                m = self.m[sl] + (f(1) - beta1) * (g - self.m[sl])
                v = f(self.beta2) * self.v[sl] + (f(1) - f(self.beta2)) * g * g
                self.m[sl], self.v[sl] = m, v
                w[sl] = w[sl] * (f(1) - lr * decay) - (lr / bc1) * m / (np.sqrt(v) / np.sqrt(bc2) + f(self.eps))
        self.step += 1
        return w
