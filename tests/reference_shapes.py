"""Stand-ins for the layer classes of the reference's model scripts (test infrastructure).

The reference's scripts cannot be imported here (``transformer.py`` imports ``deepspeed`` at module scope), so
these small modules rebuild the *structure* those scripts give their layers -- attribute names, registration order
and forward arithmetic of ``EncoderLayer`` / ``LayerNorm`` (DeepSpeedExamples/pipeline_parallelism/
transformer.py:77-172), ``DecoderLayerSimple`` (gpt2.py:20-34) and ``BottleNeck`` (resnet.py:49-75) -- so that ``state_dict()`` keys, their order and the
forward results are the reference's.  They are torch-autograd modules: the parity oracle for what this package
takes over from such modules."""
import math

import torch
from torch import nn


class RefLayerNorm(nn.Module):
    def __init__(self, features, eps=1e-6):
        super().__init__()
        self.a_2 = nn.Parameter(torch.ones(features))
        self.b_2 = nn.Parameter(torch.zeros(features))
        self.eps = eps

    def forward(self, x):
        mu, sd = x.mean(-1, keepdim=True), x.std(-1, keepdim=True)
        return self.a_2 * (x - mu) / (sd + self.eps) + self.b_2


class RefSublayer(nn.Module):
    def __init__(self, size, p):
        super().__init__()
        self.norm = RefLayerNorm(size)
        self.dropout = nn.Dropout(p)

    def forward(self, x, fn):
        return x + self.dropout(fn(self.norm(x)))


class RefAttention(nn.Module):
    def __init__(self, h, d_model, p=0.1):
        super().__init__()
        self.d_k, self.h = d_model // h, h
        self.linears = nn.ModuleList([nn.Linear(d_model, d_model) for _ in range(4)])
        self.dropout = nn.Dropout(p)

    def forward(self, q, k, v, mask=None):
        b = q.size(0)
        q, k, v = [lin(t).view(b, -1, self.h, self.d_k).transpose(1, 2) for lin, t in zip(self.linears, (q, k, v))]
        s = q @ k.transpose(-2, -1) / math.sqrt(self.d_k)
        if mask is not None:
            s = s.masked_fill(mask.unsqueeze(1) == 0, -1e9)
        y = self.dropout(s.softmax(-1)) @ v
        return self.linears[3](y.transpose(1, 2).contiguous().view(b, -1, self.h * self.d_k))


class RefFeedForward(nn.Module):
    def __init__(self, d_model, d_ff, p=0.1):
        super().__init__()
        self.w_1, self.w_2 = nn.Linear(d_model, d_ff), nn.Linear(d_ff, d_model)
        self.dropout = nn.Dropout(p)

    def forward(self, x):
        return self.w_2(self.dropout(torch.relu(self.w_1(x))))


class RefEncoderLayer(nn.Module):
    def __init__(self, size, heads, d_ff, dropout):
        super().__init__()
        self.self_attn = RefAttention(heads, size, dropout)
        self.feed_forward = RefFeedForward(size, d_ff, dropout)
        self.sublayer = nn.ModuleList([RefSublayer(size, dropout) for _ in range(2)])
        self.size = size

    def forward(self, x, mask=None):
        x = self.sublayer[0](x, lambda t: self.self_attn(t, t, t, mask))
        return self.sublayer[1](x, self.feed_forward)


class RefDecoderLayer(nn.Module):
    """Structure of ``DecoderLayerSimple`` (gpt2.py:20-34): attribute names and registration order self_attn, src_attn,
    feed_forward, sublayer[0..2]; the memory of the second attention is sqrt(1 - x) of the layer's input."""

    def __init__(self, size, heads, d_ff, dropout):
        super().__init__()
        self.size = size
        self.self_attn = RefAttention(heads, size, dropout)
        self.src_attn = RefAttention(heads, size, dropout)
        self.feed_forward = RefFeedForward(size, d_ff, dropout)
        self.sublayer = nn.ModuleList([RefSublayer(size, dropout) for _ in range(3)])

    def forward(self, x):
        m = torch.sqrt(1 - x)
        x = self.sublayer[0](x, lambda t: self.self_attn(t, t, t))
        x = self.sublayer[1](x, lambda t: self.src_attn(t, m, m))
        return self.sublayer[2](x, self.feed_forward)


class RefBottleNeck(nn.Module):
    def __init__(self, cin, cmid, stride=1, eps=1e-5):
        super().__init__()
        co = 4 * cmid
        self.residual_function = nn.Sequential(
            nn.Conv2d(cin, cmid, 1, bias=False), nn.BatchNorm2d(cmid, eps=eps), nn.ReLU(),
            nn.Conv2d(cmid, cmid, 3, stride=stride, padding=1, bias=False), nn.BatchNorm2d(cmid, eps=eps), nn.ReLU(),
            nn.Conv2d(cmid, co, 1, bias=False), nn.BatchNorm2d(co, eps=eps))
        self.shortcut = nn.Sequential()
        if stride != 1 or cin != co:
            self.shortcut = nn.Sequential(nn.Conv2d(cin, co, 1, stride=stride, bias=False), nn.BatchNorm2d(co, eps=eps))

    def forward(self, x):
        return torch.relu(self.residual_function(x) + self.shortcut(x))
