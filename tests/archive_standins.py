"""Stand-ins for the reference's scripted modules, for archives this test suite writes itself: the same attribute
names, held the same way (plain tensor attributes, sub-modules in ModuleLists; matmul.py:12,67-68,144-201,
block.py:13-47, layernorm.py:4-10, emb.py:4-6, opt.py:31-48), with trivial forwards.  Built from the CPU oracle's
quantiser, so that what a reader gets back can be compared with known values."""
from typing import List

import torch

from oracle import rwkv_oracle as O


class MM8Like(torch.nn.Module):
    def __init__(self, w):
        super().__init__()
        self.device = "cpu"
        self.stream = False
        self.runtimedtype = torch.float64
        self.weight, self.range, self.offset = O.quantize_matrix(w.float())
        self.M = int(self.weight.shape[0])
        self.N = int(self.weight.shape[1])

    def forward(self, y):
        return (y * self.range).to(torch.float32) @ self.weight.to(torch.float32) + (y * self.offset).sum()


class MM8x3Like(MM8Like):
    def __init__(self, w, w1, w2):
        super().__init__(w)
        self.weight1, self.range1, self.offset1 = O.quantize_matrix(w1.float())
        self.weight2, self.range2, self.offset2 = O.quantize_matrix(w2.float())

    def forward(self, y):
        return (y * self.range1).to(torch.float32) @ self.weight1.to(torch.float32) + (y * self.offset2).sum()


class LinearLike(torch.nn.Module):
    def __init__(self, *mods):
        super().__init__()
        self.w = torch.tensor(0)                     # what delw() leaves behind (matmul.py:171-172)
        self.weights = torch.nn.ModuleList(list(mods))
        self.device = "cpu"
        self.runtimedtype = torch.float64

    def forward(self, x):
        out = torch.zeros(1)
        for w in self.weights:
            out = out + w(x).sum()
        return out


class LayerNormLike(torch.nn.Module):
    def __init__(self, weight, bias):
        super().__init__()
        self.weight = weight.clone().to(torch.float64)
        self.bias = bias.clone().to(torch.float64)
        self.device = torch.device("cpu")
        self.runtimedtype = torch.float64

    def forward(self, x):
        return self.weight * x.to(self.device) + self.bias


class EmbLike(torch.nn.Module):
    def __init__(self, w):
        super().__init__()
        self.w = w.clone()

    def forward(self, x):
        return self.w[x].to(torch.float64)


class BlockLike(torch.nn.Module):
    def __init__(self, w, i: int):
        super().__init__()
        p = f"blocks.{i}."
        self.t: List[int] = []
        self.ln1 = LayerNormLike(w[p + "ln1.weight"], w[p + "ln1.bias"])
        self.ln2 = LayerNormLike(w[p + "ln2.weight"], w[p + "ln2.bias"])
        self.att = LinearLike(MM8x3Like(w[p + "att.key.weight"], w[p + "att.value.weight"], w[p + "att.receptance.weight"]))
        self.ffnkey = LinearLike(MM8Like(w[p + "ffn.key.weight"]))
        self.ffnvalue = LinearLike(MM8Like(w[p + "ffn.value.weight"]))
        self.attout = LinearLike(MM8Like(w[p + "att.output.weight"]))
        self.ffnreceptance = LinearLike(MM8Like(w[p + "ffn.receptance.weight"]))
        self.attmix = torch.stack((w[p + "att.time_mix_k"].squeeze(), w[p + "att.time_mix_v"].squeeze(),
                                   w[p + "att.time_mix_r"].squeeze())).unsqueeze(1).to(torch.float64).clone()
        self.time_first = w[p + "att.time_first"].squeeze().to(torch.float64).clone()
        self.time_decay = w[p + "att.time_decay"].squeeze().double().exp().neg().clone().to(torch.float64)
        self.ffnmix = torch.stack((w[p + "ffn.time_mix_k"].squeeze(),
                                   w[p + "ffn.time_mix_r"].squeeze())).unsqueeze(1).to(torch.float64).clone()

    def forward(self, x):
        return self.ln2(self.ln1(x)) * self.time_first + self.attout(x) + self.att(x) + self.ffnkey(x)


class ModelLike(torch.nn.Module):
    def __init__(self, w, dims: int, layers: int):
        super().__init__()
        self.emptyState = torch.tensor(layers * [[[0.0] * dims] * 4 + [[-1e30] * dims]], dtype=torch.float64)
        self.emb = EmbLike(w["emb.weight"])
        self.ln_out = LayerNormLike(w["ln_out.weight"], w["ln_out.bias"])
        self.ln_in = LayerNormLike(w["blocks.0.ln0.weight"], w["blocks.0.ln0.bias"])
        self.head = LinearLike(MM8Like(w["head.weight"]))
        self.blocks = torch.nn.ModuleList([BlockLike(w, i) for i in range(layers)])

    def forward(self, x):
        y = self.ln_in(self.emb(x))
        for b in self.blocks:
            y = b(y)
        return self.head(self.ln_out(y))


def write_archive(sd, path: str) -> None:
    dims = len(sd["blocks.0.att.key.weight"])
    layers = len([k for k in sd if "blocks" in k and "ln1.bias" in k])
    torch.jit.save(torch.jit.script(ModelLike(sd, dims, layers).eval()), path)
