"""The restated PCF-NAT / MFA-NAT callers against vectors written by the reference's own model
code (tests/golden/make_model_golden.py): same state_dict, same inputs -> same embeddings.
The attention itself runs through the CPU oracle here (the product has no CPU path); what this
pins is everything around the operator - head split/merge, grouped projections, block
composition, sinusoid table, pooling with lengths, parameter names."""
import os

import pytest
import torch

from oracle import na1d_oracle as O
from na1d_amd import models

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
COMMON = dict(frames=24, patch_size=2, in_chans=10, output_emb_size=16, embed_dim=32, depths=[2, 2],
              drop_path_rate=0.1, proj_channel=24, asp=True, poolnorm=True, dtype=torch.float32)
CASES = {
    "pcf": (models.PCF_NATransformer, dict(num_heads=[[4, 2], [4, 4]], win_size=[[5, 0], [[6, 2], 5]], groups=[2, 1])),
    "mfa": (models.MFA_NATransformer, dict(num_heads=[[4, 4], [4, 2]], win_size=[[5, [6, 2]], [5, 0]])),
}


def oracle_na(q, k, v, W, L, rpb=None, t_valid=None, num_heads=1):
    T = q.shape[1]
    pad = None if t_valid is None else (T - t_valid).to(torch.int64)
    return O.na1d_forward(q, k, v, W, L, rpb.reshape(num_heads, W), pad, num_heads)[0]


@pytest.mark.parametrize("name", sorted(CASES))
def test_model_reproduces_reference_vectors(name):
    cls, extra = CASES[name]
    blob = torch.load(os.path.join(GOLD, "model_%s.pt" % name), weights_only=True)
    model = cls(**COMMON, **extra, na=oracle_na)
    missing, unexpected = model.load_state_dict(blob["state_dict"], strict=True), None
    model.eval()
    with torch.no_grad():
        out_lens = model(blob["x"], blob["lens"])
        out_full = model(blob["x"])
    assert torch.allclose(out_lens, blob["out_lens"], atol=2e-5, rtol=1e-4)
    assert torch.allclose(out_full, blob["out_full"], atol=2e-5, rtol=1e-4)
    assert not torch.allclose(blob["out_lens"], blob["out_full"], atol=1e-3)      # the lengths matter


def test_state_dict_names_match_reference():
    blob = torch.load(os.path.join(GOLD, "model_pcf.pt"), weights_only=True)
    cls, extra = CASES["pcf"]
    ours = cls(**COMMON, **extra, na=oracle_na).state_dict()
    assert list(ours.keys()) == list(blob["state_dict"].keys())
    assert all(ours[k].shape == v.shape for k, v in blob["state_dict"].items())
    assert "blocks.0.blocks.0.attn.relative_position_bias" in ours and "blocks.0.blocks.0.attn.attn_mask" in ours


def test_full_size_layer_counts():
    """configs/pcf_nat4x4.yaml, pcf_nat6x4.yaml, mfa_nat4x4.yaml: 14 NA + 2 global layers (4x4), 22 + 2 (6x4)."""
    def count(m):
        layers = [l for b in m.blocks for l in b.blocks]
        return sum(l.local for l in layers), sum(not l.local for l in layers)
    assert count(models.PCF_NATransformer()) == (14, 2)
    assert count(models.MFA_NATransformer()) == (14, 2)
    assert count(models.pcf_nat_6x4()) == (22, 2)
    att = models.PCF_NATransformer().blocks[0].blocks[0].attn
    assert (att.win_size, att.left, att.num_heads, att.dim // att.num_heads) == (27, 13, 16, 16)


def test_first_step_loss_matches_published_log():
    """results/mfa_nat4x4/epoch=1/loss_log.txt:1 records a first-step loss of 17.77 with 17 982 classes:
    with random embeddings the AAM sub-centre loss sits near ln(n) + s*(margin terms) ~ 17-19."""
    torch.manual_seed(0)
    head = models.ArcMarginSubCenters(192, 17982, m=0.2, s=32.0, subcenters=3)
    loss, _ = head(torch.randn(256, 192), torch.randint(0, 17982, (256,)))
    assert 16.0 < loss.item() < 20.0


@pytest.mark.parametrize("groups", [1, 2, 4, 8])
def test_token_major_projections_equal_the_grouped_convolutions(groups):
    """The fused_qkv path runs the channels-first 1x1 convolutions as matrix products with reordered rows; the
    result must be the reference's head split (PCF_NATransformer.py:126-139) / the plain output projection."""
    torch.manual_seed(groups)
    n, dim, t, heads = 2, 64, 11, 4
    layer = models.NAttention(t, dim, heads, 7, groups=groups, channels_first=True, na="fused_qkv")
    x = torch.randn(n, dim, t)
    want = models._split_heads(layer.qkv(x), heads, groups, True)                       # [3, N*H, T, hd]
    order = models._qkv_channel_order(dim, groups, x.device)
    wq = models._dense_weight(layer.qkv).index_select(0, order).t().unsqueeze(0).expand(n, -1, -1)
    qkv = torch.baddbmm(layer.qkv.bias.index_select(0, order).view(1, 1, -1), x.transpose(1, 2), wq)
    got = qkv.view(n, t, 3, heads, dim // heads).permute(2, 0, 3, 1, 4).reshape(3, n * heads, t, dim // heads)
    assert torch.allclose(got, want, atol=1e-5)
    o = torch.randn(n, t, dim)
    wp = models._dense_weight(layer.proj).unsqueeze(0).expand(n, -1, -1)
    got = torch.baddbmm(layer.proj.bias.view(1, -1, 1), wp, o.transpose(1, 2))
    assert got.is_contiguous() and torch.allclose(got, layer.proj(o.transpose(1, 2)), atol=1e-5)


def _random_stats(module, seed=0):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, buf in module.named_buffers():
            if name.endswith("running_mean"):
                buf.copy_(torch.randn(buf.shape, generator=g) * 0.3)
            if name.endswith("running_var"):
                buf.copy_(torch.rand(buf.shape, generator=g) + 0.5)
        for p in module.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.2)


@pytest.mark.parametrize("groups", [1, 4])
def test_token_major_inference_pieces_equal_the_channels_first_modules(groups):
    """The inference pipeline's restructured pieces (batch norms folded into the neighbouring projections, the
    pooling's context never concatenated) against the plain modules, in fp32 on the CPU."""
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        embed = models.PatchEmbed(8, 16, 2, groups, True).eval()
        _random_stats(embed, 1)
        x = torch.randn(3, 8, 21, generator=g)
        assert torch.allclose(embed.forward_tokens(x), embed(x).transpose(1, 2), atol=1e-5)

        pre, block = models.BatchNorm1d(16).eval(), models.TDNNBlock(16, 24, 1).eval()
        _random_stats(pre, 2), _random_stats(block, 3)
        h = torch.randn(3, 16, 10, generator=g)
        assert torch.allclose(block.forward_tokens(h.transpose(1, 2), pre_norm=pre), block(pre(h)).transpose(1, 2), atol=1e-5)
        assert torch.allclose(block.forward_tokens(h.transpose(1, 2)), block(h).transpose(1, 2), atol=1e-5)

        pool = models.AttentiveStatisticsPooling(24, attention_channels=8).eval()
        _random_stats(pool, 4)
        z = torch.randn(3, 24, 10, generator=g)
        for lens in (None, torch.tensor([1.0, 0.5, 0.8])):
            assert torch.allclose(pool.forward_tokens(z.transpose(1, 2).contiguous(), lens), pool(z, lens), atol=1e-5)
        plain = models.StatisticsPooling()
        assert torch.allclose(plain.forward_tokens(z.transpose(1, 2).contiguous(), None), plain(z, None))


def test_training_mode_uses_the_fixed_length_mask():
    """The reference's NAttention adds its constructor-time mask (full length, nothing padded) while training and
    rebuilds the mask from `padding` only in eval mode (models/PCF_NATransformer.py:131-134)."""
    torch.manual_seed(3)
    layer = models.NAttention(frames=40, dim=32, num_heads=2, win_size=7, groups=1, channels_first=True,
                              dtype=torch.float32, na=oracle_na)
    x = torch.randn(3, 32, 40)
    pad = torch.tensor([0, 9, 25])
    layer.train()
    assert torch.equal(layer(x, padding=pad), layer(x, padding=None))
    layer.eval()
    with torch.no_grad():
        masked, plain = layer(x, padding=pad), layer(x, padding=None)
    assert torch.equal(masked[0], plain[0]) and not torch.allclose(masked[1:], plain[1:])
