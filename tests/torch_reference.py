"""TEST INFRASTRUCTURE -- float64 torch-functional forward passes of the five architectures, written from
the architecture descriptions alone (BERT: post-LN, erf-GELU, additive mask; ConvBERT: mixed attention with
span-based dynamic convolution, kernel 9; GPT-NeoX: rotary embedding on a quarter of each head, causal mask,
parallel residual; EfficientNet-B0: MBConv with squeeze-excite and swish; VGG-16).

They take the weights from a generated graph's initializers in creation order, asserting each one's shape, and
know nothing else about the graph.  tests/test_oracle_graphs.py uses them to pin the oracle's graph runner and
the graph generators on small instances; tests/test_gpu_full_size.py uses them as the exactly-rounded value
that both the oracle (sequential fp32 sums) and the GPU (blocked fp32 sums) approximate.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F


class Params:
    """The float initializers of rank >= 1 in creation order, handed out one by one as float64 tensors.
    With `randomize_seed` the generators' all-zero biases and all-one scales are first overwritten in place with
    random values, so that a bias or scale wired to the wrong place (or dropped) changes the result."""

    def __init__(self, net, randomize_seed=None):
        rng = np.random.Generator(np.random.PCG64(randomize_seed)) if randomize_seed is not None else None
        self.items = []
        for v in net.initializers:
            c = v.const
            if c.dtype != np.float32 or c.ndim == 0:
                continue
            if rng is not None and c.size > 1 and (not c.any() or (c == 1).all()):
                c[...] = rng.standard_normal(c.shape).astype(np.float32) * np.float32(0.5) + (1 if c.flat[0] == 1 else 0)
            self.items.append(c)
        self.at = 0

    def take(self, *shape):
        c = self.items[self.at]
        self.at += 1
        assert tuple(c.shape) == tuple(shape), f"initializer {self.at - 1}: shape {c.shape}, architecture wants {shape}"
        return torch.from_numpy(c.astype(np.float64))

    def done(self):
        assert self.at == len(self.items), f"{len(self.items) - self.at} float initializers were never used"


def _gelu(x):
    return x * 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))


def _swish(x):
    return x * torch.sigmoid(x)

def _attention(q, k, v, heads, bias=None, causal=False):
    """q, k, v [1, S, heads*d] -> context [1, S, heads, d]"""
    S, d = q.shape[1], q.shape[2] // heads
    qh, kh, vh = (t.view(1, S, heads, d).permute(0, 2, 1, 3) for t in (q, k, v))
    s = qh @ kh.transpose(-1, -2) / math.sqrt(d)
    if bias is not None:
        s = s + bias
    if causal:
        s = torch.where(torch.tril(torch.ones(S, S, dtype=torch.bool)), s, torch.tensor(torch.finfo(torch.float32).min, dtype=s.dtype))
    return (torch.softmax(s, -1) @ vh).permute(0, 2, 1, 3)


def _embeddings(p, feeds, vocab, types, hidden, seq, eps):
    ids = torch.from_numpy(feeds["input_ids"])
    tok = torch.from_numpy(feeds["token_type_ids"])
    word, typ, pos = p.take(vocab, hidden), p.take(types, hidden), p.take(1, seq, hidden)
    x = word[ids] + typ[tok] + pos
    return F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)



def bert(net, feeds, seq, layers, hidden, heads, ffn, vocab, eps=1e-12, randomize_seed=None):
    p = Params(net, randomize_seed)
    x = _embeddings(p, feeds, vocab, 2, hidden, seq, eps)
    bias = (1.0 - torch.from_numpy(feeds["attention_mask"]).double())[:, None, None, :] * -10000.0
    for _ in range(layers):
        q = x @ p.take(hidden, hidden) + p.take(hidden)
        k = x @ p.take(hidden, hidden) + p.take(hidden)
        v = x @ p.take(hidden, hidden) + p.take(hidden)
        c = _attention(q, k, v, heads, bias).reshape(1, seq, hidden)
        o = c @ p.take(hidden, hidden) + p.take(hidden)
        x = F.layer_norm(o + x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(x @ p.take(hidden, ffn) + p.take(ffn))
        f = h @ p.take(ffn, hidden) + p.take(hidden)
        x = F.layer_norm(f + x, (hidden,), p.take(hidden), p.take(hidden), eps)
    p.done()
    return x


def convbert(net, feeds, seq, layers, hidden, heads, ffn, vocab, eps=1e-12, ck=9, randomize_seed=None):
    p = Params(net, randomize_seed)
    nh = heads // 2
    hd = hidden // heads
    inner = nh * hd
    x = _embeddings(p, feeds, vocab, 2, hidden, seq, eps)
    bias = (1.0 - torch.from_numpy(feeds["attention_mask"]).double())[:, None, None, :] * -10000.0
    for _ in range(layers):
        q = x @ p.take(hidden, inner) + p.take(inner)
        k = x @ p.take(hidden, inner) + p.take(inner)
        v = x @ p.take(hidden, inner) + p.take(inner)
        # separable convolution of the layer input over the sequence: depthwise k=9 (no bias), pointwise (+ bias)
        dw = F.conv1d(x.transpose(1, 2), p.take(hidden, 1, ck), None, padding=ck // 2, groups=hidden)
        key_conv = F.conv1d(dw, p.take(inner, hidden, 1), p.take(inner)).transpose(1, 2)
        conv_attn = key_conv * q
        kernel = conv_attn @ p.take(inner, nh * ck) + p.take(nh * ck)
        kernel = torch.softmax(kernel.reshape(seq * nh, ck, 1), dim=1)
        conv_out = x @ p.take(hidden, inner) + p.take(inner)
        windows = F.pad(conv_out, (0, 0, ck // 2, ck // 2)).unfold(1, ck, 1)        # [1, S, inner, k]
        conv_out = (windows.reshape(seq * nh, hd, ck) @ kernel).reshape(1, seq, nh, hd)
        c = torch.cat([_attention(q, k, v, nh, bias), conv_out], dim=2).reshape(1, seq, hidden)
        o = c @ p.take(hidden, hidden) + p.take(hidden)
        x = F.layer_norm(o + x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(x @ p.take(hidden, ffn) + p.take(ffn))
        f = h @ p.take(ffn, hidden) + p.take(hidden)
        x = F.layer_norm(f + x, (hidden,), p.take(hidden), p.take(hidden), eps)
    p.done()
    return x


def gpt_neox(net, feeds, seq, layers, hidden, heads, ffn, vocab, eps=1e-5, randomize_seed=None):
    p = Params(net, randomize_seed)
    hd = hidden // heads
    rot = hd // 4
    x = p.take(vocab, hidden)[torch.from_numpy(feeds["input_ids"])]
    # rotary tables, base 10000, over the first quarter of each head; the graph's constants must equal them
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    ang = torch.arange(seq, dtype=torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    cos, sin = p.take(1, 1, seq, rot), p.take(1, 1, seq, rot)
    assert torch.allclose(cos[0, 0], emb.cos(), atol=1e-6, rtol=0) and torch.allclose(sin[0, 0], emb.sin(), atol=1e-6, rtol=0)
    cos, sin = cos[0, 0], sin[0, 0]  # the float32-rounded tables the graph holds

    def rotary(t):  # [1, heads, S, hd]
        t_rot, t_pass = t[..., :rot], t[..., rot:]
        half = torch.cat([-t_rot[..., rot // 2:], t_rot[..., : rot // 2]], dim=-1)
        return torch.cat([t_rot * cos + half * sin, t_pass], dim=-1)

    keep = torch.tril(torch.ones(seq, seq, dtype=torch.bool))
    for _ in range(layers):
        a_in = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
        qkv = (a_in @ p.take(hidden, 3 * hidden) + p.take(3 * hidden)).view(1, seq, heads, 3 * hd)
        q, k, v = (qkv[..., i * hd:(i + 1) * hd].permute(0, 2, 1, 3) for i in range(3))
        q, k = rotary(q), rotary(k)
        s = (q @ k.transpose(-1, -2)) * (1.0 / math.sqrt(hd))
        s = torch.where(keep, s, torch.tensor(float(np.finfo(np.float32).min), dtype=s.dtype))
        c = (torch.softmax(s, -1) @ v).permute(0, 2, 1, 3).reshape(1, seq, hidden)
        attn = c @ p.take(hidden, hidden) + p.take(hidden)
        m_in = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
        h = _gelu(m_in @ p.take(hidden, ffn) + p.take(ffn))
        mlp = h @ p.take(ffn, hidden) + p.take(hidden)
        x = mlp + attn + x
    x = F.layer_norm(x, (hidden,), p.take(hidden), p.take(hidden), eps)
    logits = x @ p.take(hidden, vocab)
    p.done()
    return logits


_B0_STAGES = [(1, 3, 1, 16, 1), (6, 3, 2, 24, 2), (6, 5, 2, 40, 2), (6, 3, 2, 80, 3), (6, 5, 1, 112, 3), (6, 5, 2, 192, 4),
              (6, 3, 1, 320, 1)]


def efficientnet_b0(net, feeds, classes=1000, div=1, randomize_seed=None):
    p = Params(net, randomize_seed)

    def ch(c):
        return max(4, c // div)

    def conv(x, cout, k, stride, groups=1):
        cin = x.shape[1]
        return F.conv2d(x, p.take(cout, cin // groups, k, k), p.take(cout), stride=stride, padding=(k - 1) // 2, groups=groups)

    x = _swish(conv(torch.from_numpy(feeds["input"]).double(), ch(32), 3, 2))
    for expand, k, stride, cout, repeats in _B0_STAGES:
        for r in range(repeats):
            inp, cin = x, x.shape[1]
            mid = cin * expand
            h = _swish(conv(x, mid, 1, 1)) if expand != 1 else x
            h = _swish(conv(h, mid, k, stride if r == 0 else 1, groups=mid))
            se = h.mean(dim=(2, 3), keepdim=True)
            se = _swish(conv(se, max(1, cin // 4), 1, 1))
            se = torch.sigmoid(conv(se, mid, 1, 1))
            h = conv(h * se, ch(cout), 1, 1)
            x = h + inp if h.shape == inp.shape and (r > 0 or stride == 1) else h
    x = _swish(conv(x, ch(1280), 1, 1)).mean(dim=(2, 3))
    logits = x @ p.take(classes, x.shape[1]).T + p.take(classes)
    p.done()
    return logits


def vgg16(net, feeds, classes=1000, div=1, fc=4096, randomize_seed=None):
    p = Params(net, randomize_seed)
    x = torch.from_numpy(feeds["input"]).double()
    for item in [64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M"]:
        if item == "M":
            x = F.max_pool2d(x, 2, 2)
        else:
            cout = max(4, item // div)
            x = F.relu(F.conv2d(x, p.take(cout, x.shape[1], 3, 3), p.take(cout), padding=1))
    x = x.flatten(1)
    for i, n in enumerate([fc // div, fc // div, classes]):
        x = x @ p.take(n, x.shape[1]).T + p.take(n)
        if i < 2:
            x = F.relu(x)
    p.done()
    return x
