"""One tiny module per op, following the shapes of the reference's llcompiler/test_models/ops/*.py."""
import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["Add", "Sub", "Mul", "Div", "Abs", "Relu", "ElewiseFusion1", "Matmul", "BatchMatmul", "Linear", "Conv2D_NCHW_FCHW",
           "MaxPool2D", "ReduceFusion1", "Where", "Transpose", "Slice", "BatchNorm2D_Inference", "LayerNorm", "Softmax", "Gelu",
           "Extract", "Embedding", "Braodcast", "Unsqueeze", "RecudeMax", "RecudeSum", "Sqrt", "Exp", "EQ", "Drop",
           "BatchNorm1D_Inference", "Decompose_BatchNorm", "Where3", "Slice2", "Extract3", "MaxPool2D_Twice"]


class Add(nn.Module):
    def forward(self, x):
        x = x + x
        return x + 3


class Sub(nn.Module):
    def forward(self, x):
        return (x - 3) - x * 0.5


class Mul(nn.Module):
    def forward(self, x):
        return x * x * 2


class Div(nn.Module):
    def forward(self, x):
        return x / 2 / (x * x + 1)


class Abs(nn.Module):
    def forward(self, x):
        return torch.abs(x)


class Relu(nn.Module):
    def forward(self, x):
        return F.relu(x)


class ElewiseFusion1(nn.Module):
    """x+x; -3; /2; relu; * x   (the chain timed in the reference's elementwise-fusion notes)"""

    def forward(self, x):
        y = x + x
        y = y - 3
        y = y / 2
        y = F.relu(y)
        return y * x


class Matmul(nn.Module):
    def forward(self, x, y):
        return torch.matmul(x, y)


class BatchMatmul(nn.Module):
    def forward(self, x, y):
        return torch.bmm(x, y.transpose(-1, -2))


class Linear(nn.Module):
    def __init__(self, n_in=1000):
        super().__init__()
        self.l1, self.l2, self.l3 = nn.Linear(n_in, 10), nn.Linear(10, 100), nn.Linear(100, 10)

    def forward(self, x):
        return self.l3(self.l2(self.l1(x)))


class Conv2D_NCHW_FCHW(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(3, 10, kernel_size=5, stride=1, padding=2, bias=False)
        self.conv2 = nn.Conv2d(10, 3, kernel_size=5, stride=1, padding=2, bias=True)

    def forward(self, x):
        return self.conv2(self.conv(x))


class MaxPool2D(nn.Module):
    def __init__(self):
        super().__init__()
        self.pool = nn.MaxPool2d(kernel_size=5, stride=1, padding=2, dilation=2)

    def forward(self, x):
        return self.pool(x)


class ReduceFusion1(nn.Module):
    """softmax over the last dim followed by an elementwise tail"""

    def forward(self, x):
        return torch.softmax(x + x, -1) * 2


class Where(nn.Module):
    def forward(self, x, y):
        return torch.where(x > y, x, y * 2)


class Transpose(nn.Module):
    def forward(self, x):
        return x.permute(0, 2, 1, 3).contiguous() + 1


class Slice(nn.Module):
    def forward(self, x):
        return x[:, 1:3, ::2] * 2


class Extract(nn.Module):
    def forward(self, x):
        return x[1] + x[-1]


class BatchNorm2D_Inference(nn.Module):
    def __init__(self, c=3):
        super().__init__()
        self.bn = nn.BatchNorm2d(c)
        gen = torch.Generator().manual_seed(0)
        self.bn.running_mean.data = torch.randn(c, generator=gen)
        self.bn.running_var.data = torch.rand(c, generator=gen) + 0.5
        self.bn.weight.data = torch.randn(c, generator=gen)
        self.bn.bias.data = torch.randn(c, generator=gen)

    def forward(self, x):
        return self.bn(x)


class LayerNorm(nn.Module):
    def __init__(self, n=96):
        super().__init__()
        self.ln = nn.LayerNorm(n, eps=1e-5)

    def forward(self, x):
        return self.ln(x)


class Softmax(nn.Module):
    def forward(self, x):
        return torch.softmax(x, -1)


class Gelu(nn.Module):
    def forward(self, x):
        return F.gelu(x)


class Embedding(nn.Module):
    def __init__(self, n=50, d=32):
        super().__init__()
        self.emb = nn.Embedding(n, d)

    def forward(self, idx):
        return self.emb(idx) * 2


# ---- the remaining modules of the reference's llcompiler/test_models/ops/*.py, by behaviour (names as there) ----
class Braodcast(nn.Module):
    """A [M,N] tensor added to itself viewed as [1,M,N] and as [M,1,N] (braodcast.py: rank-extending broadcasts)."""

    def forward(self, x):
        a = x + x.reshape(1, x.shape[0], x.shape[1])
        b = x + x.reshape(x.shape[0], 1, x.shape[1])
        return a + b


class Unsqueeze(nn.Module):
    def forward(self, x):
        return x.unsqueeze(1) + x.unsqueeze(1)


class RecudeMax(nn.Module):
    """amax over dim rank-of-batch-1 with and without keepdim (squeezed), then over the last dim (reduce.py)."""

    def forward(self, x):
        d = x.shape[0] - 1
        y = x.amax(d, keepdim=False) + x.amax(d, keepdim=True).squeeze(d)
        return y.amax(-1, keepdim=True)


class RecudeSum(nn.Module):
    def forward(self, x):
        d = x.shape[0] - 1
        y = x.sum(d, keepdim=False) + x.sum(d, keepdim=True).squeeze(d)
        return y.sum(-1, keepdim=True)


class Sqrt(nn.Module):
    def forward(self, x):
        return x.sqrt()          # NaN for negative inputs, in eager and compiled alike


class Exp(nn.Module):
    def forward(self, x):
        return x.exp()


class EQ(nn.Module):
    def forward(self, x):
        return (x == x) == 2     # a bool compared with 2: all False


class Drop(nn.Module):
    def __init__(self):
        super().__init__()
        self.drop = nn.Dropout()

    def forward(self, x):
        return self.drop(x)      # identity in inference


class BatchNorm1D_Inference(nn.Module):
    def __init__(self, c=3):
        super().__init__()
        self.bn = nn.BatchNorm1d(c)
        gen = torch.Generator().manual_seed(1)
        self.bn.running_mean.data = torch.randn(c, generator=gen)
        self.bn.running_var.data = torch.rand(c, generator=gen) + 0.5

    def forward(self, x):
        for _ in range(4):
            x = self.bn(x)
        return x


class Decompose_BatchNorm(nn.Module):
    """linear -> batch norm -> relu, twice, then flatten (decompose.py)."""

    def __init__(self):
        super().__init__()
        self.l1, self.b1 = nn.Linear(224, 100), nn.BatchNorm1d(100)
        self.l2, self.b2 = nn.Linear(100, 10), nn.BatchNorm1d(10)

    def forward(self, x):
        x = F.relu(self.b1(self.l1(x)))
        x = F.relu(self.b2(self.l2(x)))
        return torch.flatten(x, 1)


class Where3(nn.Module):
    """where.py: x.where(pred, y) + y with the predicate as an input."""

    def forward(self, pred, x, y):
        return x.where(pred, y) + y


class Slice2(nn.Module):
    def forward(self, x):
        return x[0:3] + x[3:6]


class Extract3(nn.Module):
    def forward(self, x):
        return x[1] + x[-2] + x[0]


class MaxPool2D_Twice(nn.Module):
    def __init__(self):
        super().__init__()
        self.pool = nn.MaxPool2d(5, 1, 2, 2)

    def forward(self, x):
        return self.pool(self.pool(x))
