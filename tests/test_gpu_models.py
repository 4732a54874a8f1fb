"""The three model-level configurations (PCF-NAT 4x4 inference, PCF-NAT 6x4 variable length, MFA-NAT 4x4 training
step) at reduced batch: the GPU models (HIP operator, 16-bit autocast) against a CPU fp32
twin with the same state_dict whose attention is the oracle.  Bars: embedding cosine >= 0.999."""
import pytest
import torch
import torch.nn.functional as F

from oracle import na1d_oracle as O
from na1d_amd import models

pytestmark = pytest.mark.gpu


def oracle_na(q, k, v, W, L, rpb=None, t_valid=None, num_heads=1, dilation=1):
    T = q.shape[1]
    pad = None if t_valid is None else (T - t_valid).to(torch.int64)
    return O.na1d_forward(q, k, v, W, L, rpb.reshape(num_heads, W), pad, num_heads, dilation=dilation)[0]


def _randomise_norm_stats(model, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for k, v in model.state_dict().items():
            if k.endswith("running_mean"):
                v.copy_(torch.randn(v.shape, generator=g) * 0.1)
            if k.endswith("running_var"):
                v.copy_(torch.rand(v.shape, generator=g) * 0.5 + 0.75)


def _twin(factory, dtype, seed=0, **kw):
    torch.manual_seed(seed)
    cpu = factory(na=oracle_na, dtype=dtype, **kw)
    _randomise_norm_stats(cpu, seed)
    return cpu


@pytest.mark.parametrize("na", ["fused", "fused_qkv", "unfused"])
def test_pcf_nat_4x4_inference_bf16(na):
    """cfg3: 80-dim fbank, 200 frames, bf16; pooled speaker embedding vs the CPU twin."""
    cpu = _twin(models.PCF_NATransformer, torch.bfloat16).eval()
    gpu = models.PCF_NATransformer(na=na, dtype=torch.bfloat16)
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.cuda().eval()
    x = torch.randn(8, 80, 200, generator=torch.Generator().manual_seed(1))
    x = x - x.mean(-1, keepdim=True)                       # CMN over time, as the evaluation harness does
    with torch.no_grad():
        want = cpu(x)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = gpu(x.cuda())
    cos = F.cosine_similarity(got.float().cpu(), want, dim=-1)
    assert got.shape == (8, 192)
    assert cos.min().item() >= 0.999, cos


@pytest.mark.parametrize("na", ["fused", "fused_qkv"])
def test_dilated_pcf_nat_bf16(na):
    """The dilation argument of the model (models/PCF_NATransformer.py:323,333,373: an int or one per block),
    which the reference can only run on the CPU: per-layer dilations 1..3 (1 for the global layers) and
    variable lengths."""
    kw = dict(dilation=[[2, 1], 2, [3, 1], [2, 3]], depths=(2, 2, 2, 2))
    cpu = _twin(models.PCF_NATransformer, torch.bfloat16, **kw).eval()
    gpu = models.PCF_NATransformer(na=na, dtype=torch.bfloat16, **kw)
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.cuda().eval()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 80, 240, generator=g)
    lens = torch.tensor([1.0, 0.8, 0.55, 0.9])
    with torch.no_grad():
        want = cpu(x, lens)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = gpu(x.cuda(), lens.cuda())
    cos = F.cosine_similarity(got.float().cpu(), want, dim=-1)
    assert cos.min().item() >= 0.999, cos


@pytest.mark.parametrize("na", ["fused", "fused_qkv"])
def test_pcf_nat_6x4_variable_length_bf16(na):
    """cfg4: lengths uniform in 300..2000 frames, padded to the longest, masks from `lens`."""
    cpu = _twin(models.pcf_nat_6x4, torch.bfloat16).eval()
    gpu = models.pcf_nat_6x4(na=na, dtype=torch.bfloat16)
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.cuda().eval()
    g = torch.Generator().manual_seed(2)
    frames = torch.randint(300, 2001, (4,), generator=g)
    tmax = int(frames.max())
    x = torch.randn(4, 80, tmax, generator=g)
    for i, f in enumerate(frames):
        x[i, :, f:] = 0
    lens = frames.float() / tmax
    with torch.no_grad():
        want = cpu(x, lens)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = gpu(x.cuda(), lens.cuda())
    cos = F.cosine_similarity(got.float().cpu(), want, dim=-1)
    assert cos.min().item() >= 0.999, cos


@pytest.mark.parametrize("na", ["fused", "fused_qkv"])
def test_mfa_nat_4x4_training_step_fp16(na):
    """cfg5: forward+backward through NA1D under fp16 autocast with a GradScaler, AAM sub-centre head over
    5994 classes, one SGD-Nesterov step; loss and parameter gradients vs the CPU fp32 twin."""
    cpu = _twin(models.MFA_NATransformer, torch.float16, frames=200).train()
    gpu = models.MFA_NATransformer(na=na, dtype=torch.float16, frames=200)
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.cuda().train()
    torch.manual_seed(3)
    head_cpu = models.ArcMarginSubCenters(192, 5994, m=0.2, s=32.0, subcenters=3)
    head_gpu = models.ArcMarginSubCenters(192, 5994, m=0.2, s=32.0, subcenters=3)
    head_gpu.load_state_dict(head_cpu.state_dict())
    head_gpu = head_gpu.cuda()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(8, 80, 200, generator=g)
    labels = torch.randint(0, 5994, (8,), generator=g)

    loss_cpu, _ = head_cpu(cpu(x), labels)
    loss_cpu.backward()

    opt = torch.optim.SGD(list(gpu.parameters()) + list(head_gpu.parameters()), lr=0.01, momentum=0.9, nesterov=True)
    scaler = torch.amp.GradScaler("cuda", init_scale=1024.0)
    with torch.autocast("cuda", dtype=torch.float16):
        emb = gpu(x.cuda())
    loss_gpu, _ = head_gpu(emb.float(), labels.cuda())
    scaler.scale(loss_gpu).backward()
    scaler.unscale_(opt)
    assert abs(loss_gpu.item() - loss_cpu.item()) < 0.05 * abs(loss_cpu.item())
    checked = 0
    for (name, pc), pg in zip(cpu.named_parameters(), gpu.parameters()):
        if pc.grad is None or pc.grad.norm() < 1e-6:
            continue
        if any(s in name for s in ("relative_position_bias", "qkv.weight", "fc.weight", "patch_embed.proj.weight")):
            cos = F.cosine_similarity(pg.grad.float().cpu().flatten(), pc.grad.flatten(), dim=0).item()
            assert cos > 0.98, (name, cos)
            checked += 1
    assert checked >= 20
    before = gpu.fc.weight.detach().clone()
    scaler.step(opt)
    scaler.update()
    assert not torch.equal(before, gpu.fc.weight.detach())


@pytest.mark.parametrize("na", ["fused", "fused_qkv", "unfused"])
def test_attention_dropout_in_training_only(na):
    """attn_drop / drop of the reference's constructors (models/PCF_NATransformer.py:324,375; 0 in its
    configurations): inactive in eval mode; in training the fused layers drop probabilities inside the kernels,
    the un-fused chain between its two calls as the reference does (:149)."""
    kw = dict(depths=(2, 2), num_heads=[[16, 4], [16, 16]], win_size=[[27, 0], [27, 27]], groups=(8, 4))
    torch.manual_seed(0)
    plain = models.PCF_NATransformer(dtype=torch.bfloat16, na=na, **kw)
    drop = models.PCF_NATransformer(dtype=torch.bfloat16, na=na, attn_drop=0.2, drop=0.1, **kw)
    drop.load_state_dict(plain.state_dict())
    plain, drop = plain.cuda(), drop.cuda()
    x = torch.randn(4, 80, 200, generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(plain.eval()(x), drop.eval()(x))
    x300 = torch.randn(4, 80, 300, generator=torch.Generator().manual_seed(2)).cuda()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        a, b = drop.train()(x300), drop(x300)
    assert torch.isfinite(a).all() and not torch.equal(a, b)         # two draws of the masks
    a.float().sum().backward()
    g = drop.blocks[0].blocks[0].attn.qkv.weight.grad
    assert g is not None and torch.isfinite(g).all() and g.abs().sum() > 0


def test_dilated_layer_drops_in_training_only():
    """A dilated layer (the reference runs these on the CPU only, models/PCF_NATransformer.py:158-170) with
    attn_drop: eval is the plain layer, training draws a fresh mask per call and has finite gradients."""
    torch.manual_seed(3)
    layer = models.NAttention(frames=90, dim=64, num_heads=4, win_size=15, groups=1, channels_first=True, na="fused",
                              dilation=3, attn_drop=0.25).cuda().to(torch.bfloat16)
    plain = models.NAttention(frames=90, dim=64, num_heads=4, win_size=15, groups=1, channels_first=True, na="fused",
                              dilation=3).cuda().to(torch.bfloat16)
    plain.load_state_dict(layer.state_dict())
    x = torch.randn(3, 64, 90, generator=torch.Generator().manual_seed(4)).cuda().to(torch.bfloat16).requires_grad_(True)
    with torch.no_grad():
        assert torch.equal(layer.eval()(x), plain.eval()(x))
    a, b = layer.train()(x), layer(x)
    assert torch.isfinite(a).all() and not torch.equal(a, b)
    a.float().sum().backward()
    assert torch.isfinite(x.grad).all() and x.grad.abs().sum() > 0


@pytest.mark.parametrize("na", ["fused", "fused_qkv"])
def test_mfa_nat_4x4_inference_with_lengths_fp16(na):
    """The tokens-first family in inference (fused_qkv: the token-major pipeline with folded batch norms, the
    global layers masked from the lengths) against the CPU fp32 twin."""
    cpu = _twin(models.MFA_NATransformer, torch.float16, seed=4).eval()
    gpu = models.MFA_NATransformer(na=na, dtype=torch.float16)
    gpu.load_state_dict(cpu.state_dict())
    gpu = gpu.cuda().eval()
    g = torch.Generator().manual_seed(6)
    x = torch.randn(5, 80, 260, generator=g)
    lens = torch.tensor([1.0, 0.7, 0.45, 0.9, 0.62])
    with torch.no_grad():
        want = cpu(x, lens)
        with torch.autocast("cuda", dtype=torch.float16):
            got = gpu(x.cuda(), lens.cuda())
    cos = F.cosine_similarity(got.float().cpu(), want, dim=-1)
    assert cos.min().item() >= 0.999, cos


def test_model_trains_under_torch_compile():
    """na="fused_op": the attention layers call the registered ops, so the whole model compiles into one graph
    (fullgraph) and a training step gives the eager step's loss and gradients."""
    kw = dict(depths=(2, 2), num_heads=[[16, 4], [16, 16]], win_size=[[27, 0], [27, 27]], groups=(8, 4), frames=120)
    torch.manual_seed(0)
    eager = models.PCF_NATransformer(dtype=torch.bfloat16, na="fused", **kw).cuda().train()
    comp = models.PCF_NATransformer(dtype=torch.bfloat16, na="fused_op", **kw).cuda().train()
    comp.load_state_dict(eager.state_dict())
    step = torch.compile(comp, backend="aot_eager", fullgraph=True)
    x = torch.randn(16, 80, 120, generator=torch.Generator().manual_seed(1)).cuda()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        a, b = eager(x), step(x)
    assert F.cosine_similarity(a.float(), b.float(), dim=-1).min() > 0.999
    a.float().pow(2).sum().backward()
    b.float().pow(2).sum().backward()
    checked = 0
    for (name, p), q in zip(eager.named_parameters(), comp.parameters()):
        if not (name.endswith("weight") or "relative_position_bias" in name):
            continue                     # a bias in front of a batch norm has an exactly zero gradient: noise both ways
        if p.grad is not None and p.grad.norm() > 1e-6:
            assert F.cosine_similarity(p.grad.flatten().float(), q.grad.flatten().float(), dim=0) > 0.97, name
            checked += 1                 # two bf16 runs through differently decomposed batch norms
    assert checked > 30


def test_inference_replayed_from_a_captured_graph():
    """GraphedInference: one capture per input shape, then replays - with lengths as a graph input, eager passes and
    synchronisations between the replays, and every replay checked against the eager result (some library ops record
    nodes that do not replay faithfully; the class verifies, and so does this test, on fresh inputs)."""
    from na1d_amd.graphs import GraphedInference
    kw = dict(depths=(2, 2), num_heads=[[16, 4], [16, 16]], win_size=[[27, 0], [27, 27]], groups=(8, 4))
    torch.manual_seed(0)
    model = models.PCF_NATransformer(dtype=torch.bfloat16, na="fused_qkv", **kw).cuda().eval()
    _randomise_norm_stats(model, 3)
    g = torch.Generator().manual_seed(9)
    x0 = torch.randn(6, 80, 260, generator=g).cuda()
    lens0 = torch.tensor([1.0, 0.8, 0.5, 0.9, 0.65, 0.72]).cuda()
    graphed = GraphedInference(model, x0, lens0)
    for i in range(4):
        x = torch.randn(6, 80, 260, generator=g).cuda()
        lens = (0.4 + 0.6 * torch.rand(6, generator=g)).cuda()
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            want = model(x, lens)
        torch.cuda.synchronize()
        got = graphed(x, lens).clone()
        torch.cuda.synchronize()
        assert F.cosine_similarity(got.float(), want.float(), dim=-1).min() > 0.9999, i
        assert (got - want).abs().max() <= 0.05 * want.abs().max()
    with pytest.raises(AssertionError):
        graphed(x[:3], lens[:3])                                # another shape needs another capture


def _small_pcf(use_checkpoint, attn_drop, na):
    torch.manual_seed(11)
    m = models.PCF_NATransformer(frames=120, embed_dim=64, depths=(2, 2), num_heads=[[4, 1], [4, 4]],
                                 win_size=[[9, 0], [[8, 3], 9]], groups=[2, 1], proj_channel=96, output_emb_size=32,
                                 drop_path_rate=0.0, attn_drop=attn_drop, use_checkpoint=use_checkpoint,
                                 dtype=torch.float16, na=na)
    return m.cuda().train()


@pytest.mark.parametrize("na", ["fused", "fused_qkv", "unfused"])
@pytest.mark.parametrize("attn_drop", [0.0, 0.2])
def test_training_with_activation_checkpointing_reenters_the_operator(na, attn_drop):
    """The reference trains PCF-NAT 6x4 with activation checkpointing (configs/pcf_nat6x4.yaml:62): the layer's
    forward, and with it the operator's, runs a second time inside backward (models/PCF_NATransformer.py:298-299).
    One training step with checkpointing must give the loss and the gradients of the same step without it, bit
    for bit - also with attention dropout, whose mask the recomputation has to draw again identically."""
    if na == "unfused" and attn_drop > 0:
        pytest.skip("torch's dropout in the two-call chain draws from the GPU generator; covered by torch itself")
    x = torch.randn(6, 80, 120, generator=torch.Generator().manual_seed(12)).cuda()
    results = []
    for ckpt in (False, True):
        model = _small_pcf(ckpt, attn_drop, na)
        torch.manual_seed(13)                       # the seeds of the attention dropout are drawn from here
        with torch.autocast("cuda", dtype=torch.float16):
            emb = model(x)
        loss = emb.float().square().mean()
        loss.backward()
        results.append((loss.detach().clone(), [p.grad.detach().clone() for p in model.parameters() if p.grad is not None]))
    (l0, g0), (l1, g1) = results
    assert torch.equal(l0, l1) and len(g0) == len(g1) > 10
    rpb_like = 0
    for a, b in zip(g0, g1):
        if a.dim() == 4 and a.shape[0] == 1 and a.shape[2] == 1:       # d rpb is summed with float atomics
            assert torch.allclose(a, b, rtol=1e-3, atol=1e-6)
            rpb_like += 1
        else:
            assert torch.equal(a, b)
    assert rpb_like >= 3 and all(g.abs().max() > 0 for g in g0)


def test_pcf_nat_6x4_full_batch_agrees_with_the_checked_small_batch():
    """cfg4 at its full size (64 utterances, 300..2000 frames, padded to the longest): a sample's embedding does
    not depend on what else is in the batch, so the first and last four samples of the full batch must reproduce
    an eight-sample batch padded to the same length - the size test_pcf_nat_6x4_variable_length_bf16 holds
    against the CPU twin."""
    torch.manual_seed(0)
    gpu = models.pcf_nat_6x4(na="fused_qkv", dtype=torch.bfloat16).cuda().eval()
    g = torch.Generator().manual_seed(2)
    frames = torch.randint(300, 2001, (64,), generator=g)
    frames[0] = 2000                                   # both batches are padded to 2000 frames
    tmax = int(frames.max())
    x = torch.randn(64, 80, tmax, generator=g)
    for i, f in enumerate(frames):
        x[i, :, f:] = 0
    lens = frames.float() / tmax
    pick = list(range(4)) + list(range(60, 64))
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        full = gpu(x.cuda(), lens.cuda())
        small = gpu(x[pick].cuda(), lens[pick].cuda())
    assert full.shape == (64, 192) and torch.isfinite(full).all()
    cos = F.cosine_similarity(full[pick].float(), small.float(), dim=-1)
    assert cos.min().item() >= 0.9999, cos


def test_mfa_nat_4x4_full_batch_training_step_agrees_with_the_checked_small_batch():
    """cfg5 at its full size (batch 128 x 200 frames, fp16 autocast): in training mode batch norm couples the
    samples, so the full-size step is held against the small one where it can be - in eval mode the embeddings of
    the first eight samples equal those of an eight-sample batch; in training mode the full step runs, its loss
    is close to ln(5994) + s * sin(m)-ish for random weights and every gradient is finite and non-zero."""
    torch.manual_seed(0)
    gpu = models.MFA_NATransformer(na="fused_qkv", dtype=torch.float16, frames=200).cuda()
    head = models.ArcMarginSubCenters(192, 5994, m=0.2, s=32.0, subcenters=3).cuda()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(128, 80, 200, generator=g).cuda()
    labels = torch.randint(0, 5994, (128,), generator=g).cuda()
    gpu.eval()
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
        full, small = gpu(x), gpu(x[:8])
    assert F.cosine_similarity(full[:8].float(), small.float(), dim=-1).min().item() >= 0.9999
    gpu.train()
    scaler = torch.amp.GradScaler("cuda", init_scale=1024.0)
    with torch.autocast("cuda", dtype=torch.float16):
        emb = gpu(x)
    loss, _ = head(emb.float(), labels)
    scaler.scale(loss).backward()
    assert 6.0 < loss.item() < 30.0
    grads = [p.grad for p in gpu.parameters() if p.grad is not None]
    assert len(grads) > 100 and all(torch.isfinite(gr).all() for gr in grads)
    assert sum(float(gr.abs().max() > 0) for gr in grads) > 0.9 * len(grads)
