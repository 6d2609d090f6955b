"""The benchmark configurations as plain torch modules with seeded random-init weights."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def _normal_(module, std=0.02, seed=0):
    gen = torch.Generator().manual_seed(seed)
    for p in module.parameters():
        if p.dim() >= 2:
            p.data = torch.randn(p.shape, generator=gen) * std
        else:
            p.data.zero_()
    return module


class MLP(nn.Module):
    """Config 1: [4,784] -> Linear 784->512 -> ReLU -> Linear 512->10; weights N(0,0.02), biases zero."""

    def __init__(self, seed=0):
        super().__init__()
        self.fc1 = nn.Linear(784, 512)
        self.fc2 = nn.Linear(512, 10)
        _normal_(self, 0.02, seed)

    def forward(self, x):
        return self.fc2(F.relu(self.fc1(x)))


def make_mlp_inputs(batch=4, seed=1):
    return (torch.randn(batch, 784, generator=torch.Generator().manual_seed(seed)),)


class _ConvAct(nn.Module):
    """Conv with BatchNorm already folded in (so: conv with bias), optional ReLU."""

    def __init__(self, cin, cout, k, stride, pad, relu=True):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, k, stride, pad, bias=True)
        self.relu = relu

    def forward(self, x):
        y = self.conv(x)
        return F.relu(y) if self.relu else y


class _BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.c1 = _ConvAct(cin, cout, 3, stride, 1, relu=True)
        self.c2 = _ConvAct(cout, cout, 3, 1, 1, relu=False)
        self.down = _ConvAct(cin, cout, 1, stride, 0, relu=False) if (stride != 1 or cin != cout) else None

    def forward(self, x):
        idt = x if self.down is None else self.down(x)
        return F.relu(self.c2(self.c1(x)) + idt)


class ResNet18Folded(nn.Module):
    """Config 3: ResNet-18-style CNN, NCHW fp32, BatchNorm folded into the convolutions: 7x7/2 stem,
    3x3/2 max-pool, four stages of two basic blocks (64/128/256/512), global average pool, FC 512->1000.
    Kaiming-normal (fan_out, relu) conv weights; the folded biases are small seeded values so that the
    bias path is exercised."""

    def __init__(self, num_classes=1000, seed=0):
        super().__init__()
        self.stem = _ConvAct(3, 64, 7, 2, 3)
        chans = [64, 128, 256, 512]
        blocks, cin = [], 64
        for i, c in enumerate(chans):
            blocks += [_BasicBlock(cin, c, 1 if i == 0 else 2), _BasicBlock(c, c, 1)]
            cin = c
        self.blocks = nn.Sequential(*blocks)
        self.fc = nn.Linear(512, num_classes)
        gen = torch.Generator().manual_seed(seed)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                fan_out = m.out_channels * m.kernel_size[0] * m.kernel_size[1]
                m.weight.data = torch.randn(m.weight.shape, generator=gen) * math.sqrt(2.0 / fan_out)
                m.bias.data = torch.randn(m.bias.shape, generator=gen) * 0.05
            elif isinstance(m, nn.Linear):
                m.weight.data = torch.randn(m.weight.shape, generator=gen) * 0.02
                m.bias.data.zero_()

    def forward(self, x):
        x = self.stem(x)
        x = F.max_pool2d(x, 3, 2, 1)
        x = self.blocks(x)
        x = F.adaptive_avg_pool2d(x, 1).flatten(1)
        return self.fc(x)


class _ConvBN(nn.Module):
    """Conv without bias followed by BatchNorm2d (the torchvision unit), optional ReLU."""

    def __init__(self, cin, cout, k, stride, pad, relu=True):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, k, stride, pad, bias=False)
        self.bn = nn.BatchNorm2d(cout)
        self.relu = relu

    def forward(self, x):
        y = self.bn(self.conv(x))
        return F.relu(y) if self.relu else y


class _BasicBlockBN(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.c1 = _ConvBN(cin, cout, 3, stride, 1, relu=True)
        self.c2 = _ConvBN(cout, cout, 3, 1, 1, relu=False)
        self.down = _ConvBN(cin, cout, 1, stride, 0, relu=False) if (stride != 1 or cin != cout) else None

    def forward(self, x):
        idt = x if self.down is None else self.down(x)
        return F.relu(self.c2(self.c1(x)) + idt)


class ResNet18BN(nn.Module):
    """The same network as ResNet18Folded the way torchvision spells it: every convolution has no bias and is
    followed by a BatchNorm2d.  In eval mode the compiler folds each batch norm into its convolution when the plan
    is made.  The affine parameters and the running statistics are seeded random values (variances in [0.5, 1.5]),
    so the fold is not the identity."""

    def __init__(self, num_classes=1000, seed=0):
        super().__init__()
        self.stem = _ConvBN(3, 64, 7, 2, 3)
        chans = [64, 128, 256, 512]
        blocks, cin = [], 64
        for i, c in enumerate(chans):
            blocks += [_BasicBlockBN(cin, c, 1 if i == 0 else 2), _BasicBlockBN(c, c, 1)]
            cin = c
        self.blocks = nn.Sequential(*blocks)
        self.fc = nn.Linear(512, num_classes)
        gen = torch.Generator().manual_seed(seed)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                fan_out = m.out_channels * m.kernel_size[0] * m.kernel_size[1]
                m.weight.data = torch.randn(m.weight.shape, generator=gen) * math.sqrt(2.0 / fan_out)
            elif isinstance(m, nn.BatchNorm2d):
                m.weight.data = 0.75 + 0.5 * torch.rand(m.weight.shape, generator=gen)
                m.bias.data = torch.randn(m.bias.shape, generator=gen) * 0.05
                m.running_mean.copy_(torch.randn(m.running_mean.shape, generator=gen) * 0.1)
                m.running_var.copy_(0.5 + torch.rand(m.running_var.shape, generator=gen))
            elif isinstance(m, nn.Linear):
                m.weight.data = torch.randn(m.weight.shape, generator=gen) * 0.02
                m.bias.data.zero_()

    def forward(self, x):
        x = self.stem(x)
        x = F.max_pool2d(x, 3, 2, 1)
        x = self.blocks(x)
        x = F.adaptive_avg_pool2d(x, 1).flatten(1)
        return self.fc(x)


def make_resnet_inputs(batch=16, size=224, seed=1):
    return (torch.randn(batch, 3, size, size, generator=torch.Generator().manual_seed(seed)),)


class _SelfAttention(nn.Module):
    def __init__(self, hidden, heads):
        super().__init__()
        self.heads, self.dh = heads, hidden // heads
        self.q, self.k, self.v, self.o = (nn.Linear(hidden, hidden) for _ in range(4))

    def forward(self, x, mask=None):
        B, S, H = x.shape
        def split(t):
            return t.view(B, S, self.heads, self.dh).permute(0, 2, 1, 3)
        q, k, v = split(self.q(x)), split(self.k(x)), split(self.v(x))
        scores = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(self.dh)
        if mask is not None:
            scores = scores + mask
        p = torch.softmax(scores, dim=-1)
        ctx = torch.matmul(p, v).permute(0, 2, 1, 3).reshape(B, S, H)
        return self.o(ctx)


class EncoderBlock(nn.Module):
    """Config 4: pre-LayerNorm transformer encoder block: hidden 768, 12 heads of 64, FFN 3072 with
    exact GELU, eps 1e-5, weights N(0,0.02)."""

    def __init__(self, hidden=768, heads=12, ffn=3072, seed=0):
        super().__init__()
        self.ln1, self.ln2 = nn.LayerNorm(hidden, eps=1e-5), nn.LayerNorm(hidden, eps=1e-5)
        self.attn = _SelfAttention(hidden, heads)
        self.fc1, self.fc2 = nn.Linear(hidden, ffn), nn.Linear(ffn, hidden)
        _normal_(self, 0.02, seed)
        self.ln1.weight.data.fill_(1.0)
        self.ln2.weight.data.fill_(1.0)

    def forward(self, x):
        x = x + self.attn(self.ln1(x))
        return x + self.fc2(F.gelu(self.fc1(self.ln2(x))))


def make_encoder_inputs(batch=8, seq=512, hidden=768, seed=1, dtype=torch.float32):
    return (torch.randn(batch, seq, hidden, generator=torch.Generator().manual_seed(seed)).to(dtype),)


class _BertLayer(nn.Module):
    def __init__(self, hidden, heads, ffn):
        super().__init__()
        self.attn = _SelfAttention(hidden, heads)
        self.ln1, self.ln2 = nn.LayerNorm(hidden, eps=1e-5), nn.LayerNorm(hidden, eps=1e-5)
        self.fc1, self.fc2 = nn.Linear(hidden, ffn), nn.Linear(ffn, hidden)

    def forward(self, x, mask):
        x = self.ln1(x + self.attn(x, mask))
        return self.ln2(x + self.fc2(F.gelu(self.fc1(x))))


class BertEncoder(nn.Module):
    """Config 5: BERT-base-shaped post-LayerNorm encoder stack (embeddings left out: the input is the
    embedded sequence), additive attention mask [B,1,1,S] with 0 / -1e4 entries."""

    def __init__(self, layers=12, hidden=768, heads=12, ffn=3072, seed=0):
        super().__init__()
        self.layers = nn.ModuleList(_BertLayer(hidden, heads, ffn) for _ in range(layers))
        _normal_(self, 0.02, seed)
        for l in self.layers:
            l.ln1.weight.data.fill_(1.0)
            l.ln2.weight.data.fill_(1.0)

    def forward(self, x, mask):
        for l in self.layers:
            x = l(x, mask)
        return x


def make_bert_inputs(batch=8, seq=128, hidden=768, seed=1):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, seq, hidden, generator=gen)
    lengths = torch.randint(seq // 2, seq + 1, (batch,), generator=gen)
    mask = torch.zeros(batch, 1, 1, seq)
    for b in range(batch):
        mask[b, :, :, int(lengths[b]):] = -1e4
    return x, mask
