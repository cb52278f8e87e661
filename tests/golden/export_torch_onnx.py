"""Writes the torch_*.onnx fixtures of this directory: small decoder pieces serialised to the ONNX
wire format by PyTorch's own (TorchScript) exporter, with inputs and the outputs PyTorch computed on
the CPU in fp32. They pin the ONNX readers (native and oracle/onnx_read.py) and whole-graph numerics
against an implementation that shares no code with this repository.

    python tests/golden/export_torch_onnx.py        # needs torch; the `onnx` package is not needed

The exporter's last step (merging onnxscript custom functions into the model) imports the `onnx`
package although these models have no such functions; that step is replaced by the identity.
"""
import io
import math
import os
import warnings

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def export(module, args, names_in, names_out, dynamic_axes=None):
    from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto
    f = io.BytesIO()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.onnx.export(module, args, f, opset_version=14, input_names=names_in,
                          output_names=names_out, dynamic_axes=dynamic_axes, dynamo=False)
    return f.getvalue()


class NormProj(torch.nn.Module):
    """RMSNorm in the x * rsqrt(mean(x^2) + eps) * g form, a projection, a softmax."""

    def __init__(self):
        super().__init__()
        g = torch.Generator().manual_seed(11)
        self.w = torch.nn.Parameter(torch.randn(64, 48, generator=g) * 0.1)
        self.g = torch.nn.Parameter(torch.rand(64, generator=g) + 0.5)

    def forward(self, x):
        v = x.pow(2).mean(-1, keepdim=True)
        y = x * torch.rsqrt(v + 1e-5) * self.g
        return torch.softmax(y @ self.w, -1)


class DecoderBlock(torch.nn.Module):
    """One Llama-style layer: RMSNorm, grouped-query attention with rotary embedding and an
    additive mask, SwiGLU MLP. Static shapes: batch 1, 6 tokens, hidden 64, 4 heads / 2 KV heads
    of 16."""
    H, KV, D, HID, FFN = 4, 2, 16, 64, 128

    def __init__(self):
        super().__init__()
        g = torch.Generator().manual_seed(12)

        def p(*shape):
            return torch.nn.Parameter(torch.randn(*shape, generator=g) * 0.08)
        self.ln1 = torch.nn.Parameter(torch.rand(self.HID, generator=g) + 0.5)
        self.ln2 = torch.nn.Parameter(torch.rand(self.HID, generator=g) + 0.5)
        self.wq, self.wk, self.wv = p(self.HID, self.H * self.D), p(self.HID, self.KV * self.D), \
            p(self.HID, self.KV * self.D)
        self.wo = p(self.H * self.D, self.HID)
        self.wg, self.wu, self.wd = p(self.HID, self.FFN), p(self.HID, self.FFN), p(self.FFN, self.HID)

    @staticmethod
    def norm(x, g):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * g

    @staticmethod
    def rope(x, cos, sin):
        h = x.shape[-1] // 2
        rot = torch.cat((-x[..., h:], x[..., :h]), dim=-1)
        return x * cos + rot * sin

    def forward(self, x, cos, sin, mask):
        s = x.shape[1]
        rep = self.H // self.KV
        h = self.norm(x, self.ln1)
        q = (h @ self.wq).reshape(1, s, self.H, self.D).transpose(1, 2)
        k = (h @ self.wk).reshape(1, s, self.KV, self.D).transpose(1, 2)
        v = (h @ self.wv).reshape(1, s, self.KV, self.D).transpose(1, 2)
        q, k = self.rope(q, cos, sin), self.rope(k, cos, sin)
        k = k[:, :, None, :, :].expand(1, self.KV, rep, s, self.D).reshape(1, self.H, s, self.D)
        v = v[:, :, None, :, :].expand(1, self.KV, rep, s, self.D).reshape(1, self.H, s, self.D)
        scores = q @ k.transpose(-1, -2) / math.sqrt(self.D) + mask
        ctx = torch.softmax(scores, -1) @ v
        x = x + ctx.transpose(1, 2).reshape(1, s, self.H * self.D) @ self.wo
        h2 = self.norm(x, self.ln2)
        return x + (torch.nn.functional.silu(h2 @ self.wg) * (h2 @ self.wu)) @ self.wd


def save(name, module, inputs, names_in, names_out, dynamic_axes=None):
    module.eval()
    with torch.no_grad():
        out = module(*inputs)
    data = export(module, tuple(inputs), names_in, names_out, dynamic_axes)
    with open(os.path.join(HERE, name + ".onnx"), "wb") as f:
        f.write(data)
    arrays = {n: t.numpy() for n, t in zip(names_in, inputs)}
    arrays[names_out[0]] = out.numpy()
    np.savez(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, len(data), "bytes;", {k: v.shape for k, v in arrays.items()})


def main():
    g = torch.Generator().manual_seed(13)
    save("torch_norm_proj_softmax", NormProj(), [torch.randn(2, 5, 64, generator=g)], ["x"], ["y"],
         {"x": {1: "seq"}})
    s, d = 6, DecoderBlock.D
    pos = torch.arange(s, dtype=torch.float32)[:, None]
    inv = 1.0 / (10000.0 ** (torch.arange(0, d // 2, dtype=torch.float32) * 2 / d))
    emb = torch.cat((pos * inv, pos * inv), dim=-1)
    cos, sin = emb.cos()[None, None], emb.sin()[None, None]
    mask = torch.triu(torch.full((s, s), float("-inf")), 1)[None, None]
    save("torch_decoder_block", DecoderBlock(),
         [torch.randn(1, s, DecoderBlock.HID, generator=g), cos, sin, mask],
         ["x", "cos", "sin", "mask"], ["y"])


if __name__ == "__main__":
    main()
