"""Writes tests/golden/model_*.pt: tiny PCF-NAT / MFA-NAT forward passes computed by the
reference's own model code on CPU (its pad/unfold branch), for the parts of the callers that
only an import can pin - the composition of the forward passes, the grouped qkv head split,
attentive statistics pooling with lengths, and the state_dict naming.

Run in the build container only (needs /root/reference):  python tests/golden/make_model_golden.py
The reference's operator module compiles CUDA at import, so a stub stands in for it; the CPU
branch of the models never calls the operator.  Only tensors are stored (inputs, lengths,
outputs and the state_dict), loaded in the tests with weights_only=True.
"""
import os
import sys
import types

import torch

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))

stub = types.ModuleType("na1d_tensorcore.nattn")
stub.getNA1dFunction = lambda C, dilation, dtype: (None, None)
pkg = types.ModuleType("na1d_tensorcore")
pkg.nattn = stub
sys.modules["na1d_tensorcore"] = pkg
sys.modules["na1d_tensorcore.nattn"] = stub
sys.path.insert(0, REF)

from models.MFA_NATransformer import MFA_NATransformer  # noqa: E402
from models.PCF_NATransformer import PCF_NATransformer  # noqa: E402

COMMON = dict(frames=24, patch_size=2, in_chans=10, output_emb_size=16, embed_dim=32, depths=[2, 2],
              drop_path_rate=0.1, proj_channel=24, asp=True, poolnorm=True, dtype=torch.float32)
CASES = {
    "pcf": (PCF_NATransformer, dict(num_heads=[[4, 2], [4, 4]], win_size=[[5, 0], [[6, 2], 5]], groups=[2, 1])),
    "mfa": (MFA_NATransformer, dict(num_heads=[[4, 4], [4, 2]], win_size=[[5, [6, 2]], [5, 0]])),
}

for name, (cls, extra) in CASES.items():
    torch.manual_seed(1234)
    model = cls(**COMMON, **extra)
    with torch.no_grad():   # make the normalisation layers and biases non-trivial
        for k, v in model.state_dict().items():
            if k.endswith("running_mean") or (k.endswith(".bias") and v.dim() == 1):
                v.copy_(torch.randn_like(v) * 0.1)
            if k.endswith("running_var"):
                v.copy_(torch.rand_like(v) * 0.5 + 0.75)
    model.eval()
    x = torch.randn(3, 10, 24)
    lens = torch.tensor([1.0, 0.75, 0.5])
    with torch.no_grad():
        out_lens = model(x, lens)
        out_full = model(x)
    blob = {"config": {}, "state_dict": {k: v.clone() for k, v in model.state_dict().items()},
            "x": x, "lens": lens, "out_lens": out_lens, "out_full": out_full}
    path = os.path.join(HERE, "model_%s.pt" % name)
    torch.save(blob, path)
    print(name, "params", sum(p.numel() for p in model.parameters()), "out", tuple(out_lens.shape),
          "bytes", os.path.getsize(path))
