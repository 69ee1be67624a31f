"""The decode step around the compressed linears on a real MI355X, through the C ABI:
grouped forwards (several matrices per launch, fused epilogues) against the C oracle,
RMSNorm and the rotary attention step against fp64 restatements (oracle/llama_oracle.py,
itself pinned against `transformers`), and the whole fused step against the torch-op step
and against the float64 decoder on the rebuilt dense weights.  Tolerances as for the
layer outputs: max|d|/max|ref| <= 1e-2, mean|d|/mean|ref| <= 1e-3 unless stated."""
import numpy as np
import pytest
import torch

from bitstack_amd import _lib
from bitstack_amd.utils import inference_utils as IU
from bitstack_amd.utils.llama_decode import LlamaShape, PROJ, SyntheticLlamaDecoder
from bitstack_amd.utils.synthetic import synthetic_layer
from oracle import bitstack_oracle as O
from oracle import c_oracle as C
from oracle import llama_oracle as LO

pytestmark = pytest.mark.gpu
MAX_REL, MEAN_REL = 1e-2, 1e-3


def dev():
    return torch.device("cuda:0")


def assert_close(got, ref, what, max_rel=MAX_REL, mean_rel=MEAN_REL):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    mx, mn = d.max() / max(np.abs(ref).max(), 1e-30), d.mean() / max(np.abs(ref).mean(), 1e-30)
    print(f"{what}: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= max_rel and mn <= mean_rel, f"{what}: max_rel={mx:.3e} mean_rel={mn:.3e}"


@pytest.fixture(params=[_lib.DECODE_AUTO, _lib.DECODE_MX], ids=["planned_kernel", "block_scaled_kernel"])
def decode_kernel_mode(request):
    """The grouped launches once as planned and once with the block-scaled kernel on every one- and two-token
    pass that it takes (so that small groups reach it too)."""
    assert _lib.lib().bs_set_decode_kernel(request.param) == 0
    yield request.param
    assert _lib.lib().bs_set_decode_kernel(_lib.DECODE_AUTO) == 0


def make_group(shapes, N, T, seed, bias=False):
    """shapes: [(I, M)]; returns (MatrixGroup on the GPU, x on the CPU, fp64 reference outputs per matrix)."""
    mats, refs, x = [], [], None
    for j, (I, M) in enumerate(shapes):
        q, u, vt, xj = synthetic_layer(M, N, I, T, seed=seed + j, signed_factors=True)
        x = xj if x is None else x
        b = torch.randn(M, generator=torch.Generator().manual_seed(seed + 50 + j)).half() * 0.05 if bias else None
        refs.append(C.forward_f64(q.numpy(), u.numpy(), vt.numpy(), x.numpy(), None if b is None else b.numpy()))
        mats.append((q.to(dev()), u.to(dev()), vt.to(dev()), None if b is None else b.to(dev())))
    return IU.MatrixGroup(mats), x, refs


GROUP_CASES = [([(3, 512), (5, 128), (2, 128)], 512, 1), ([(3, 4096), (5, 1024), (2, 1024)], 4096, 1),
               ([(2, 1024), (4, 256)], 1024, 2), ([(1, 300), (2, 77), (3, 64), (1, 512)], 1536, 3),
               ([(2, 512), (3, 256)], 1024, 4), ([(2, 512), (1, 256)], 512, 5), ([(2, 256), (2, 256)], 1024, 8),
               ([(2, 300), (3, 77), (1, 64)], 1536, 9), ([(3, 1024), (2, 256)], 4096, 16), ([(2, 200), (2, 200)], 384, 32), ([(2, 300), (1, 64)], 640, 48),
               # long stacks: 16-wave workgroups in pairs, the grid cut into even runs per matrix
               ([(32, 2048), (30, 1024), (34, 1100)], 4096, 1), ([(20, 4096), (12, 1024)], 4096, 2)]


@pytest.mark.parametrize("shapes,N,T", GROUP_CASES)
def test_group_forward_side_by_side(shapes, N, T, decode_kernel_mode):
    print(f"group forward {shapes} N={N} T={T}", flush=True)
    grp, x, refs = make_group(shapes, N, T, seed=11, bias=(T % 2 == 0))
    y = IU.bitstack_forward_group_hip(grp, x.to(dev())).cpu().numpy()
    assert y.shape == (T, sum(m for _, m in shapes)) and y.dtype == np.float16
    assert_close(y, np.concatenate(refs, axis=1), "group vs fp64")
    # and the same numbers as one bs_forward per matrix, up to the order of the fp32 partial sums
    off = 0
    for (q, u, vt, b), (_, M) in zip(grp.tensors, shapes):
        single = IU.bitstack_forward_hip(q, u, vt, x.to(dev()), b).cpu().numpy()
        assert_close(y[:, off:off + M], single, "group vs single", 2e-3, 2e-4)
        off += M


@pytest.mark.parametrize("I,M,N,T", [(3, 512, 1024, 1), (2, 4096, 4096, 1), (2, 256, 512, 6), (2, 300, 640, 12)])
def test_group_forward_residual(I, M, N, T, decode_kernel_mode):
    print(f"group residual I={I} M={M} N={N} T={T}", flush=True)
    grp, x, refs = make_group([(I, M)], N, T, seed=21)
    res = (torch.randn(T, M, generator=torch.Generator().manual_seed(2)) * 0.1).half()
    y = IU.bitstack_forward_group_hip(grp, x.to(dev()), _lib.EPI_RESIDUAL, residual=res.to(dev())).cpu().numpy()
    assert_close(y, refs[0] + res.double().numpy(), "residual vs fp64")
    plain = IU.bitstack_forward_group_hip(grp, x.to(dev())).cpu()
    assert np.array_equal(y, (res.float() + plain.float()).half().numpy())        # exactly the fp16 add of the fp16 result


@pytest.mark.parametrize("I0,I1,M,N,T", [(3, 2, 1024, 512, 1), (2, 4, 14336, 4096, 1), (2, 2, 512, 1024, 7), (2, 3, 1024, 2048, 24)])
def test_group_forward_swiglu(I0, I1, M, N, T, decode_kernel_mode):
    print(f"group swiglu I={I0},{I1} M={M} N={N} T={T}", flush=True)
    grp, x, refs = make_group([(I0, M), (I1, M)], N, T, seed=31)
    # scale so that the gate spans the non-linear range of silu
    y = IU.bitstack_forward_group_hip(grp, x.to(dev()), _lib.EPI_SWIGLU).cpu().numpy()
    assert y.shape == (T, M)
    assert_close(y, LO.silu(refs[0]) * refs[1], "swiglu vs fp64", 2e-2, 2e-3)
    both = IU.bitstack_forward_group_hip(grp, x.to(dev())).cpu()
    gate, up = both[:, :M], both[:, M:]
    want = (torch.nn.functional.silu(gate.float()).half().float() * up.float()).half().numpy()
    d = np.abs(y.astype(np.float64) - want.astype(np.float64))
    assert d.max() <= 2e-3 * max(np.abs(want).max(), 1e-30)       # same rounding points; expf differs in the last bit at most


def test_group_rejects_what_the_decode_kernel_does_not_take():
    grp, x, _ = make_group([(1, 64), (1, 64)], 512, 1, seed=1)
    with pytest.raises(RuntimeError):
        IU.bitstack_forward_group_hip(grp, torch.zeros(49, 512, dtype=torch.float16, device=dev()))   # more than 48 tokens
    grp2, _, _ = make_group([(1, 64), (1, 128)], 512, 1, seed=1)
    with pytest.raises(RuntimeError):
        IU.bitstack_forward_group_hip(grp2, x.to(dev()), _lib.EPI_SWIGLU)                               # unequal M
    with pytest.raises(RuntimeError):
        IU.bitstack_forward_group_hip(grp, x.to(dev()), _lib.EPI_RESIDUAL)                               # no residual


@pytest.mark.parametrize("T,H", [(1, 4096), (3, 512), (8, 8192), (2, 16384), (5, 264)])
def test_rmsnorm(T, H):
    print(f"rmsnorm T={T} H={H}", flush=True)
    g = torch.Generator().manual_seed(H + T)
    x = (torch.randn(T, H, generator=g) * 3).half()
    w = (1 + 0.3 * torch.randn(H, generator=g)).half()
    y = IU.rmsnorm_hip(x.to(dev()), w.to(dev()), 1e-5).cpu()
    assert_close(y.numpy(), LO.rmsnorm(x.double().numpy(), w.double().numpy(), 1e-5), "rmsnorm vs fp64", 2e-3, 5e-4)
    # the rounding points of the usual implementation: normalised value to fp16, then times the weight
    v = x.float()
    want = (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * w
    assert (y.float() - want.float()).abs().max() <= 2 * torch.finfo(torch.float16).eps * want.float().abs().max()


@pytest.mark.parametrize("B,heads,kv,max_len", [(1, 32, 8, 40), (3, 4, 2, 40), (2, 8, 8, 40), (2, 16, 2, 40), (1, 6, 2, 40),
                                                # long caches; with more than 256 (head, sequence) pairs several
                                                # query heads of a KV head share a workgroup
                                                (2, 16, 2, 1100), (1, 32, 8, 1024), (9, 32, 8, 1100), (17, 16, 8, 1024), (33, 8, 8, 1024)])
def test_attention_decode_steps(B, heads, kv, max_len):
    print(f"attention B={B} heads={heads} kv={kv} max_len={max_len}", flush=True)
    d, steps = 128, 37
    g = torch.Generator().manual_seed(heads)
    cos64, sin64 = LO.rope_tables(max_len, d, 500000.0)
    cos, sin = torch.from_numpy(cos64).half(), torch.from_numpy(sin64).half()
    kc = torch.zeros(B, kv, max_len, d, dtype=torch.float16, device=dev())
    vc = torch.zeros_like(kc)
    pos = torch.zeros(1, dtype=torch.long, device=dev())
    kref = np.zeros((B, kv, max_len, d))
    vref = np.zeros((B, kv, max_len, d))
    for p in range(steps):
        qkv = torch.randn(B, (heads + 2 * kv) * d, generator=g).half()
        out = IU.attention_decode_hip(qkv.to(dev()), kc, vc, cos.to(dev()), sin.to(dev()), pos, heads, kv).cpu().numpy()
        pos.add_(1)
        x = qkv.double().numpy()
        c, s = cos[p].double().numpy(), sin[p].double().numpy()
        for b in range(B):
            q = LO.rope(x[b, :heads * d].reshape(heads, d), c, s)
            kref[b, :, p] = LO.rope(x[b, heads * d:(heads + kv) * d].reshape(kv, d), c, s)
            vref[b, :, p] = x[b, (heads + kv) * d:].reshape(kv, d)
            # the kernel attends over the fp16 cache it wrote; follow that for the reference of later steps
            want = LO.attention_decode(q, kref[b], vref[b], p + 1).reshape(-1)
            if p in (0, 1, 15, 16, 17, steps - 1):
                assert_close(out[b], want, f"attention step {p} seq {b}", 1e-2, 2e-3)
    assert_close(kc.cpu().numpy()[:, :, :steps], kref[:, :, :steps], "k cache", 2e-3, 5e-4)
    assert np.array_equal(vc.cpu().numpy()[:, :, :steps], vref[:, :, :steps].astype(np.float16))
    assert float(kc[:, :, steps:].abs().max()) == 0.0 and float(vc[:, :, steps:].abs().max()) == 0.0


@pytest.mark.parametrize("B,heads,kv,max_len,at", [(2, 16, 2, 2048, 1500), (1, 8, 4, 1024, 1023), (1, 32, 8, 4096, 3000),
                                                   (5, 64, 8, 2048, 1500), (9, 32, 16, 1024, 1023), (3, 96, 8, 1200, 517)])
def test_attention_decode_deep_in_a_long_cache(B, heads, kv, max_len, at):
    """One step at position `at` of a cache already holding random rows."""
    print(f"attention deep B={B} heads={heads} kv={kv} max_len={max_len} at={at}", flush=True)
    d = 128
    g = torch.Generator().manual_seed(at)
    cos64, sin64 = LO.rope_tables(max_len, d, 500000.0)
    cos, sin = torch.from_numpy(cos64).half(), torch.from_numpy(sin64).half()
    kc = torch.zeros(B, kv, max_len, d, dtype=torch.float16)
    vc = torch.zeros_like(kc)
    kc[:, :, :at] = torch.randn(B, kv, at, d, generator=g).half()
    vc[:, :, :at] = torch.randn(B, kv, at, d, generator=g).half()
    kd, vd = kc.to(dev()), vc.to(dev())
    qkv = torch.randn(B, (heads + 2 * kv) * d, generator=g).half()
    pos = torch.tensor([at], dtype=torch.long, device=dev())
    out = IU.attention_decode_hip(qkv.to(dev()), kd, vd, cos.to(dev()), sin.to(dev()), pos, heads, kv).cpu().numpy()
    x = qkv.double().numpy()
    c, s_ = cos[at].double().numpy(), sin[at].double().numpy()
    for b in range(B):
        q = LO.rope(x[b, :heads * d].reshape(heads, d), c, s_)
        kref, vref = kc[b].double().numpy().copy(), vc[b].double().numpy().copy()
        kref[:, at] = LO.rope(x[b, heads * d:(heads + kv) * d].reshape(kv, d), c, s_).astype(np.float16)
        vref[:, at] = x[b, (heads + kv) * d:].reshape(kv, d)
        want = LO.attention_decode(q, kref, vref, at + 1).reshape(-1)
        assert_close(out[b], want, f"attention at {at} seq {b}", 1e-2, 2e-3)
        assert_close(kd[b, :, at].cpu().numpy(), kref[:, at], "appended k", 2e-3, 5e-4)
    if at + 1 < max_len:
        assert float(kd[:, :, at + 1:].abs().max()) == 0.0


def test_attention_position_outside_the_cache_writes_zeros_and_touches_nothing():
    kc = torch.zeros(1, 2, 8, 128, dtype=torch.float16, device=dev())
    vc = torch.zeros_like(kc)
    tab = torch.ones(8, 64, dtype=torch.float16, device=dev())
    qkv = torch.ones(1, 8 * 128, dtype=torch.float16, device=dev())
    out = IU.attention_decode_hip(qkv, kc, vc, tab, tab, torch.tensor([8], device=dev()), 4, 2)
    assert float(out.abs().max()) == 0.0 and float(kc.abs().max()) == 0.0
    # the same through the grouped-query kernel (long cache, more than 256 (head, sequence) pairs)
    kc = torch.zeros(65, 2, 1024, 128, dtype=torch.float16, device=dev())
    vc = torch.zeros_like(kc)
    tab = torch.ones(1024, 64, dtype=torch.float16, device=dev())
    qkv = torch.ones(65, 8 * 128, dtype=torch.float16, device=dev())
    out = IU.attention_decode_hip(qkv, kc, vc, tab, tab, torch.tensor([1024], device=dev()), 4, 2)
    assert float(out.abs().max()) == 0.0 and float(kc.abs().max()) == 0.0


SMALL = LlamaShape(layers=2, hidden=512, intermediate=1024, heads=4, kv_heads=2, vocab=256)


def small_config(seed=0):
    g = torch.Generator().manual_seed(seed)
    return {f"layer.{L}.{p}": int(torch.randint(1, 5, (1,), generator=g)) for L in range(SMALL.layers) for p in PROJ}


def dense_weights(model):
    """Hugging Face names -> float64 arrays, the compressed linears rebuilt in float64 by the oracle."""
    w = {"model.embed_tokens.weight": model.embed.double().cpu().numpy(), "lm_head.weight": model.lm_head.double().cpu().numpy(),
         "model.norm.weight": model.final_norm.double().cpu().numpy()}
    for L in range(model.s.layers):
        w[f"model.layers.{L}.input_layernorm.weight"] = model.norm_w[L, 0].double().cpu().numpy()
        w[f"model.layers.{L}.post_attention_layernorm.weight"] = model.norm_w[L, 1].double().cpu().numpy()
        for p in PROJ:
            m = model.lin[L][p]
            w[f"model.layers.{L}.{p}.weight"] = O.reconstruct_w_exact(m.qweight.cpu().numpy(), m.u.cpu().numpy(), m.vt.cpu().numpy())
    return w


@pytest.mark.parametrize("batch", [1, 2, 4])
def test_fused_step_at_8b_layer_widths_matches_float64_decoder(batch):
    """One decoder layer at the real Llama-3.1-8B widths (hidden 4096, intermediate 14336, 32 query / 8 KV heads), one,
    two and four sequences: the grouped launches then run on the kernels the full model runs on (q/k/v and gate/up with the RMS
    scale and SwiGLU on the block-scaled kernel at one and two tokens and on the fp16 kernel at four, the residual epilogues), against the float64 decoder
    on the float64-rebuilt weights."""
    shape = LlamaShape(layers=1, hidden=4096, intermediate=14336, heads=32, kv_heads=8, vocab=512)
    cfg = {f"layer.0.{p}": b for p, b in zip(PROJ, (3, 2, 4, 3, 2, 3, 2))}
    max_len = 16
    m = SyntheticLlamaDecoder(shape, cfg, max_len, dev(), seed=8, batch=batch)
    with torch.no_grad():
        g = torch.Generator(device=dev()).manual_seed(3)
        m.norm_w.copy_(1 + 0.2 * torch.randn(m.norm_w.shape, device=dev(), generator=g))
        m.embed.mul_(30.0)
    # the gate/up and q/k/v groups are large enough for the block-scaled kernel, at two tokens too
    gu = [(cfg["layer.0.mlp.gate_proj"], 14336), (cfg["layer.0.mlp.up_proj"], 14336)]
    assert _lib.lib().bs_decode_kernel(gu[0][0] + gu[1][0], 14336, 4096, 16, batch) == (_lib.DECODE_MX if batch <= 2 else _lib.DECODE_F16)
    w = dense_weights(m)
    orcs = [LO.LlamaOracle(w, shape.layers, shape.heads, shape.kv_heads, shape.head_dim, shape.rope_theta, shape.rms_eps, max_len)
            for _ in range(batch)]
    tokens = torch.randint(0, shape.vocab, (batch, 5), generator=torch.Generator().manual_seed(2))
    for j in range(tokens.shape[1]):
        m.token.copy_(tokens[:, j])
        m.step_fused()
        got = m.logits.float().cpu().numpy()
        for s in range(batch):
            want = orcs[s].step(int(tokens[s, j]))
            assert_close(got[s], want, f"8B widths, fused vs float64, position {j} seq {s}", 2e-2, 4e-3)


@pytest.mark.parametrize("batch", [1, 3])
def test_fused_step_matches_torch_step_and_float64_decoder(batch):
    print(f"fused decode step batch={batch}", flush=True)
    cfg = small_config()
    a = SyntheticLlamaDecoder(SMALL, cfg, 24, dev(), seed=4, batch=batch)
    b = SyntheticLlamaDecoder(SMALL, cfg, 24, dev(), seed=4, batch=batch)
    # norm weights away from one, factors large enough that the layers matter
    with torch.no_grad():
        for m in (a, b):
            g = torch.Generator(device=dev()).manual_seed(9)
            m.norm_w.copy_(1 + 0.2 * torch.randn(m.norm_w.shape, device=dev(), generator=g))
            m.embed.mul_(30.0)
    w = dense_weights(a)
    orcs = [LO.LlamaOracle(w, SMALL.layers, SMALL.heads, SMALL.kv_heads, SMALL.head_dim, SMALL.rope_theta, SMALL.rms_eps, 24)
            for _ in range(batch)]
    tokens = torch.randint(0, SMALL.vocab, (batch, 10), generator=torch.Generator().manual_seed(1))
    for j in range(tokens.shape[1]):
        a.token.copy_(tokens[:, j])
        b.token.copy_(tokens[:, j])
        a.step()
        b.step_fused()
        la, lb = a.logits.float().cpu().numpy(), b.logits.float().cpu().numpy()
        assert lb.shape == (batch, SMALL.vocab)
        for s in range(batch):
            want = orcs[s].step(int(tokens[s, j]))
            assert_close(lb[s], want, f"fused vs float64, position {j} seq {s}", 2e-2, 4e-3)
            assert_close(la[s], want, f"torch step vs float64, position {j} seq {s}", 2e-2, 4e-3)
    assert int(b.pos) == tokens.shape[1]
    assert_close(b.kcache.float().cpu().numpy(), a.kcache.float().cpu().numpy(), "k cache fused vs torch", 1e-2, 2e-3)


@pytest.mark.parametrize("batch,n", [(1, 9), (3, 17)])
def test_one_pass_prefill_matches_token_by_token_and_float64_decoder(batch, n):
    """prefill(): all prompt positions at once (rebuild + dense kernels, causal attention in
    torch) leaves the same logits, next token and KV cache as feeding the prompt position by
    position, and decode continues from it."""
    print(f"one-pass prefill batch={batch} n={n}", flush=True)
    cfg = small_config()
    a = SyntheticLlamaDecoder(SMALL, cfg, 32, dev(), seed=6, batch=batch)
    b = SyntheticLlamaDecoder(SMALL, cfg, 32, dev(), seed=6, batch=batch)
    with torch.no_grad():
        for m in (a, b):
            g = torch.Generator(device=dev()).manual_seed(3)
            m.norm_w.copy_(1 + 0.2 * torch.randn(m.norm_w.shape, device=dev(), generator=g))
            m.embed.mul_(30.0)
    prompt = torch.randint(0, SMALL.vocab, (batch, n), generator=torch.Generator().manual_seed(2)).to(dev())
    a.prefill_positions(prompt, fused=True)
    b.prefill(prompt)
    assert int(b.pos) == n == int(a.pos)
    assert_close(b.logits.float().cpu().numpy(), a.logits.float().cpu().numpy(), "logits after the prompt", 2e-2, 4e-3)
    assert_close(b.kcache[:, :, :, :n].float().cpu().numpy(), a.kcache[:, :, :, :n].float().cpu().numpy(), "k cache", 1e-2, 2e-3)
    assert_close(b.vcache[:, :, :, :n].float().cpu().numpy(), a.vcache[:, :, :, :n].float().cpu().numpy(), "v cache", 1e-2, 2e-3)
    assert float(b.kcache[:, :, :, n:].abs().max()) == 0.0
    w = dense_weights(a)
    for s_ in range(batch):
        orc = LO.LlamaOracle(w, SMALL.layers, SMALL.heads, SMALL.kv_heads, SMALL.head_dim, SMALL.rope_theta, SMALL.rms_eps, 32)
        for j in range(n):
            want = orc.step(int(prompt[s_, j]))
        assert_close(b.logits[s_].float().cpu().numpy(), want, f"prefill vs float64, seq {s_}", 2e-2, 4e-3)
    # decode goes on from the prefilled cache
    b.token.copy_(a.token)
    for _ in range(3):
        a.step_fused()
        b.step_fused()
        assert_close(b.logits.float().cpu().numpy(), a.logits.float().cpu().numpy(), "decode after prefill", 2e-2, 4e-3)
        b.token.copy_(a.token)


def test_fused_step_replays_in_a_graph():
    cfg = small_config(1)
    m = SyntheticLlamaDecoder(SMALL, cfg, 32, dev(), seed=2)
    ref = SyntheticLlamaDecoder(SMALL, cfg, 32, dev(), seed=2)
    m.token.fill_(5)
    ref.token.fill_(5)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        m.step_fused()                       # warm-up outside capture: workspaces, group argument blocks
    torch.cuda.current_stream().wait_stream(side)
    m.reset()
    m.token.fill_(5)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        m.step_fused()
    m.reset()
    m.token.fill_(5)
    for step in range(6):                    # replays interleaved with eager work, each checked
        graph.replay()
        ref.step_fused()
        torch.cuda.synchronize()
        assert torch.equal(m.logits, ref.logits), step
        assert torch.equal(m.token, ref.token) and int(m.pos) == step + 1


def test_decoder_round_trips_through_a_checkpoint(tmp_path):
    """save_checkpoint -> from_checkpoint (reference layout: sharded safetensors, config.json,
    compression_config.json) gives the same logits; a smaller memory budget loads fewer blocks."""
    cfg = {k: 3 for k in small_config()}
    a = SyntheticLlamaDecoder(SMALL, cfg, 16, dev(), seed=6)
    with torch.no_grad():
        a.norm_w.copy_(1 + 0.1 * torch.randn(a.norm_w.shape, device=dev(), generator=torch.Generator(device=dev()).manual_seed(1)))
    per_block = sum(m.memory_per_bit() for row in a.lin for m in row.values())
    dense = 2 * (a.embed.numel() + a.lm_head.numel())
    configs = [{"memory": dense + b * per_block, "layers": {k: b for k in cfg}} for b in (1, 2, 3)]
    a.save_checkpoint(str(tmp_path), compression_configs=configs, max_shard_bytes=200_000)
    full_mb = (dense + 3 * per_block) / 1024 ** 2 + 0.01
    b = SyntheticLlamaDecoder.from_checkpoint(str(tmp_path), 16, dev(), max_memory_MB=full_mb)
    small = SyntheticLlamaDecoder.from_checkpoint(str(tmp_path), 16, dev(), max_memory_MB=(dense + 2 * per_block) / 1024 ** 2 + 0.01)
    assert all(m.w_bit == 3 for row in b.lin for m in row.values())
    assert all(m.w_bit == 2 and m.u.shape[0] == 2 for row in small.lin for m in row.values())
    for tok in (5, 9, 200, 31):
        for m in (a, b, small):
            m.token.fill_(tok)
            m.step_fused()
        assert torch.equal(a.logits, b.logits)
        assert not torch.equal(a.logits, small.logits)
    assert torch.equal(a.token, b.token)


@pytest.mark.parametrize("shapes,N,T,mode", [([(3, 512), (2, 128), (2, 128)], 1024, 1, "none"),
                                              ([(2, 4096), (3, 1024), (1, 1024)], 4096, 1, "none"),
                                              ([(2, 1024), (3, 1024)], 2048, 1, "swiglu"),
                                              ([(2, 256), (1, 256)], 512, 5, "swiglu"),
                                              ([(2, 512), (3, 128)], 1024, 20, "none"),
                                              # three token tiles: more token rows than one pass of the sum of squares takes
                                              ([(2, 512), (3, 128)], 1024, 40, "none"),
                                              ([(2, 256), (2, 256)], 512, 48, "swiglu"),
                                              ([(2, 300)], 1536, 3, "none")])
def test_group_forward_with_input_rms(shapes, N, T, mode, decode_kernel_mode):
    """bs_forward_group_rms: the RMSNorm in front of the matrices without a launch of its own.  The
    caller folds the norm weight into vt; the launch scales by rsqrt(mean(x^2) + eps)."""
    print(f"group rms {shapes} N={N} T={T} {mode}", flush=True)
    g = torch.Generator().manual_seed(N + T)
    wn = (1 + 0.3 * torch.randn(N, generator=g)).half()
    x = (torch.randn(T, N, generator=g) * 4).half()                       # far from unit RMS on purpose
    eps = 1e-5
    hn = LO.rmsnorm(x.double().numpy(), wn.double().numpy(), eps)         # float64 normalised input
    mats, refs = [], []
    for j, (I, M) in enumerate(shapes):
        q, u, vt, _ = synthetic_layer(M, N, I, T, seed=40 + j, signed_factors=True)
        b = (torch.randn(M, generator=g) * 0.05).half() if j % 2 == 0 else None
        w = O.reconstruct_w_exact(q.numpy(), u.numpy(), vt.numpy())
        refs.append(hn @ w.T + (0 if b is None else b.double().numpy()))
        vt_folded = (vt.float() * wn.float().view(1, 1, -1)).half()
        mats.append((q.to(dev()), u.to(dev()), vt_folded.to(dev()), None if b is None else b.to(dev())))
    grp = IU.MatrixGroup(mats)
    if mode == "swiglu":
        y = IU.bitstack_forward_group_hip(grp, x.to(dev()), _lib.EPI_SWIGLU, rms_eps=eps).cpu().numpy()
        assert_close(y, LO.silu(refs[0]) * refs[1], "rms + swiglu vs fp64", 2e-2, 3e-3)
    else:
        y = IU.bitstack_forward_group_hip(grp, x.to(dev()), rms_eps=eps).cpu().numpy()
        assert_close(y, np.concatenate(refs, axis=1), "rms group vs fp64", 1e-2, 2e-3)


@pytest.mark.parametrize("B,V", [(1, 128256), (3, 256), (2, 4096), (1, 13), (1, 8)])
def test_argmax(B, V):
    g = torch.Generator().manual_seed(V)
    x = torch.randn(B, V, generator=g).half()
    x[0, V // 2] = x[0].max()                       # a tie: the lower index must win
    got = IU.argmax_hip(x.to(dev())).cpu()
    want = torch.tensor([int(np.argmax(r)) for r in x.float().numpy()])     # numpy: first maximum
    assert torch.equal(got, want)
    x[0, 3] = float("nan")
    got = IU.argmax_hip(x.to(dev())).cpu()
    row = x[0].float().numpy().copy(); row[3] = -np.inf
    assert int(got[0]) == int(np.argmax(row))       # NaN never wins


def test_importance_scoring_and_compression_configs(tmp_path):
    """The scoring loop on a small decoder: perplexity against the float64 decoder, one entry per
    (bit level, linear), block counts restored, and configs whose memory grows by the scored
    linear's bytes per block and which the checkpoint reader accepts."""
    from bitstack_amd.utils import checkpoint as ck
    from bitstack_amd.utils import scoring as S
    niter = 3
    cfg = {f"layer.{L}.{p}": niter for L in range(SMALL.layers) for p in PROJ}
    m = SyntheticLlamaDecoder(SMALL, cfg, 32, dev(), seed=8, batch=2)
    with torch.no_grad():
        m.embed.mul_(30.0)
    ids = torch.randint(0, SMALL.vocab, (3, 12), generator=torch.Generator().manual_seed(5))
    # perplexity of the full model against the float64 decoder
    w = dense_weights(m)
    nll = []
    for s_ in range(ids.shape[0]):
        orc = LO.LlamaOracle(w, SMALL.layers, SMALL.heads, SMALL.kv_heads, SMALL.head_dim, SMALL.rope_theta, SMALL.rms_eps, 32)
        tot = 0.0
        for j in range(ids.shape[1] - 1):
            lg = orc.step(int(ids[s_, j]))
            lg = lg - lg.max()
            tot += -(lg[int(ids[s_, j + 1])] - np.log(np.exp(lg).sum()))
        nll.append(tot / (ids.shape[1] - 1))
    want = float(np.exp(np.mean(nll)))
    got = S.eval_ppl(m, ids)
    assert abs(got - want) <= 2e-2 * want, (got, want)

    seen = []
    scores = S.score_importance(m, ids, niter, progress=lambda bit, name, ppl: seen.append((bit, name)))
    # resuming every evaluation at its linear's layer gives the very same numbers
    plain = S.score_importance(m, ids, niter, reuse_prefix=False)
    assert plain == scores
    names = [n for n, _ in S.all_linears(m)]
    assert len(names) == SMALL.layers * len(PROJ)
    assert abs(scores["original_ppl"] - got) <= 1e-6 * got
    assert [lvl["bit"] for lvl in scores["reduced_ppl"]] == [1, 2]
    for lvl in scores["reduced_ppl"]:
        assert [e["layer"] for e in lvl["ppls"]] == names and all(np.isfinite(e["ppl"]) for e in lvl["ppls"])
    assert len(seen) == 2 * len(names)
    assert all(mod.w_bit == niter for _, mod in S.all_linears(m))          # restored
    configs = S.compression_configs_for(m, scores)
    assert len(configs) == 1 + 2 * len(names)
    per_bit = {n: int(mod.memory_per_bit()) for n, mod in S.all_linears(m)}
    order = S.sort_layers_and_bits_average(scores)
    for a, b, name in zip(configs[:-1], configs[1:], order):
        assert b["memory"] - a["memory"] == per_bit[name]
        assert b["layers"][name] == a["layers"][name] + 1
    assert configs[-1]["layers"] == {n: niter for n in names}
    assert configs[-1]["memory"] == m.weight_bytes() + (m.norm_w.numel() + m.final_norm.numel()) * 2
    S.save_scores_and_configs(str(tmp_path), scores, configs)
    again = ck.read_compression_configs(str(tmp_path))
    mid = configs[len(configs) // 2]
    assert ck.retrieve_compression_config(again, mid["memory"] / 1024 ** 2 + 1e-6) == mid["layers"]


def test_whole_flow_dense_to_compressed_to_budgeted_decoder(tmp_path):
    """Dense random Llama -> from_dense (decompose on the device) -> decode against the float64
    decoder on the DENSE weights, closer with every block kept -> checkpoint round trip ->
    importance scores -> compression configs -> a decoder loaded at a memory budget."""
    from bitstack_amd.utils import checkpoint as ck
    from bitstack_amd.utils import scoring as S
    print("whole flow: dense -> compressed -> scored -> budgeted", flush=True)
    niter = 4
    g = torch.Generator().manual_seed(21)
    w = {"model.embed_tokens.weight": torch.randn(SMALL.vocab, SMALL.hidden, generator=g),
         "lm_head.weight": torch.randn(SMALL.vocab, SMALL.hidden, generator=g) * SMALL.hidden ** -0.5,
         "model.norm.weight": 1 + 0.1 * torch.randn(SMALL.hidden, generator=g)}
    for L in range(SMALL.layers):
        w[f"model.layers.{L}.input_layernorm.weight"] = 1 + 0.1 * torch.randn(SMALL.hidden, generator=g)
        w[f"model.layers.{L}.post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(SMALL.hidden, generator=g)
        for p in PROJ:
            m_, n_ = SMALL.proj_shape(p)
            w[f"model.layers.{L}.{p}.weight"] = torch.randn(m_, n_, generator=g) * n_ ** -0.5
    w = {k_: v.half().float() for k_, v in w.items()}          # what a fp16 checkpoint would hold
    model = SyntheticLlamaDecoder.from_dense(SMALL, w, niter, 16, dev())
    assert all(m.w_bit == niter and m.u.shape[0] == niter and m.name == f"layer.{L}.{p}"
               for L, row in enumerate(model.lin) for p, m in row.items())
    # every block kept brings each rebuilt weight closer to the dense one (float64 rebuild)
    for L in (0, 1):
        for p in ("self_attn.k_proj", "mlp.down_proj"):
            m = model.lin[L][p]
            dense = w[f"model.layers.{L}.{p}.weight"].double().numpy()
            errs = [np.linalg.norm(O.reconstruct_w_exact(m.qweight[:b].cpu().numpy(), m.u[:b].cpu().numpy(), m.vt[:b].cpu().numpy()) - dense)
                    / np.linalg.norm(dense) for b in range(1, niter + 1)]
            assert all(errs[i + 1] < 0.8 * errs[i] for i in range(niter - 1)) and errs[-1] < 0.2, errs
    # decode against the float64 decoder on the dense weights: the gap shrinks with the blocks
    toks = [7, 130, 22, 201, 64]
    orc = LO.LlamaOracle({k_: v.double().numpy() for k_, v in w.items()}, SMALL.layers, SMALL.heads, SMALL.kv_heads,
                         SMALL.head_dim, SMALL.rope_theta, SMALL.rms_eps, 16)
    want = [orc.step(t) for t in toks]
    gaps = []
    for b in (1, 2, 4):
        model.set_bits(b)
        model.reset()
        gap = 0.0
        for t, ref in zip(toks, want):
            model.token.fill_(t)
            model.step_fused()
            gap = max(gap, float(np.abs(model.logits[0].float().cpu().numpy() - ref).max() / np.abs(ref).max()))
        gaps.append(gap)
    print("logit gaps to the dense float64 decoder at 1, 2, 4 blocks:", gaps, flush=True)
    assert gaps[0] > gaps[1] > gaps[2] and gaps[2] < 0.5 * gaps[0], gaps
    full_logits = model.logits.clone()
    # scores and configs, then the checkpoint with them, then a budgeted load
    ids = torch.randint(0, SMALL.vocab, (2, 10), generator=torch.Generator().manual_seed(3))
    scores = S.score_importance(model, ids, niter)
    assert all(m.w_bit == niter for row in model.lin for m in row.values())
    configs = S.compression_configs_for(model, scores)
    model.save_checkpoint(str(tmp_path), compression_configs=configs, max_shard_bytes=300_000)
    back = SyntheticLlamaDecoder.from_checkpoint(str(tmp_path), 16, dev(), niter=niter)
    for t in toks:
        back.token.fill_(t)
        back.step_fused()
    assert torch.equal(back.logits, full_logits)
    mems = [c["memory"] for c in ck.read_compression_configs(str(tmp_path))]
    budget = mems[len(mems) // 2]
    cut = SyntheticLlamaDecoder.from_checkpoint(str(tmp_path), 16, dev(), max_memory_MB=budget / 1024 ** 2 + 1e-3)
    assert cut.weight_bytes() <= budget < back.weight_bytes()
    kept = {f"layer.{L}.{p}": m.w_bit for L, row in enumerate(cut.lin) for p, m in row.items()}
    assert min(kept.values()) >= 1 and max(kept.values()) <= niter and len(set(kept.values())) > 1
    for t in toks:
        cut.token.fill_(t)
        cut.step_fused()
    assert torch.isfinite(cut.logits).all() and not torch.equal(cut.logits, full_logits)
    # the running full-size decoder shrunk to that budget (blocks freed) is the decoder loaded at
    # it, and grown back (blocks read from disk) it is the full one again
    full_bytes = back.weight_bytes()
    freed, loaded = back.set_memory_budget(str(tmp_path), max_memory_MB=budget / 1024 ** 2 + 1e-3)
    assert freed > 0 and loaded == 0 and back.weight_bytes() == cut.weight_bytes() == full_bytes - freed
    back.reset()
    for t in toks:
        back.token.fill_(t)
        back.step_fused()
    assert torch.equal(back.logits, cut.logits)
    freed2, loaded2 = back.set_memory_budget(str(tmp_path), compression_config={k_: niter for k_ in kept})
    assert freed2 == 0 and loaded2 == freed and back.weight_bytes() == full_bytes
    back.reset()
    for t in toks:
        back.token.fill_(t)
        back.step_fused()
    assert torch.equal(back.logits, full_logits)
