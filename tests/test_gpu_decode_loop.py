"""The decode loop (``fast_decode.greedy_decode_fast``) on a small random-weight Llama: per-step
logits against (1) a plain fp32 restatement of the model step whose attention is the oracle's
three-zone attention over the same packed bytes, and (2) the model's own ``forward`` over its
dense prompt cache (loose: K is quantized to 8 bits there); eager and HIP-graph runs must give
the same tokens; observers, EOS and error paths follow fast_decode.py:731-1137."""
import numpy as np
import pytest
import torch

from oracle import rdkv_oracle as O
from rdkv_amd import fast_decode, packing
from tests.gpu_util import DEV, require_gpu, t2n

pytestmark = pytest.mark.gpu

T_PROMPT, H_Q, H_KV, D, HID, LAYERS, VOCAB = 300, 4, 2, 128, 512, 2, 1000


def _build_setup():
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(hidden_size=HID, intermediate_size=1024, num_hidden_layers=LAYERS, num_attention_heads=H_Q,
                      num_key_value_heads=H_KV, head_dim=D, vocab_size=VOCAB, max_position_embeddings=4096,
                      rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False)
    torch.manual_seed(1234)
    model = LlamaForCausalLM(cfg)
    with torch.no_grad():           # wider weights than the default init so that logits are not flat
        for p in model.parameters():
            if p.dim() == 2:
                p.mul_(3.0)
    model = model.half().to(DEV).eval()
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, VOCAB, (1, T_PROMPT), generator=g).to(DEV)
    with torch.no_grad():
        pre = model(prompt, use_cache=True)
    kv = []
    for i in range(LAYERS):
        layer = pre.past_key_values.layers[i]
        kv.append((layer.keys.contiguous(), layer.values.contiguous()))
    return model, prompt, pre, kv


@pytest.fixture(scope="module")
def setup():
    require_gpu()
    return _build_setup()


def _pack(kv, v_bits, k_bits):
    layers, v16 = [], []
    for K, V in kv:
        pl, nvo = packing.pack_layer_per_head(K, V, v_bits, k_bits, H_Q // H_KV)
        layers.append(pl)
        v16.append(nvo)
    return packing.TriZoneCache(tuple(layers), v16, [None] * len(kv), [None] * len(kv), T_PROMPT)


def _mixed_bits(seed):
    g = torch.Generator().manual_seed(seed)
    v_bits = torch.tensor([0, 2, 4, 8, 16])[torch.randint(0, 5, (H_KV, T_PROMPT), generator=g)]
    k_bits = torch.tensor([0, 2, 4, 8])[torch.randint(0, 4, (H_KV, D), generator=g)]
    return v_bits, k_bits


def _rms(x, w, eps):
    return w * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


def _reference_logits(model, kv, v_bits, k_bits, tokens, position0):
    """fp32 CPU step of the same model, attention = oracle over oracle-packed layers.  For an
    fp16 model every intermediate is rounded to fp16 where the GPU loop stores one."""
    cfg = model.config
    if next(model.parameters()).dtype == torch.float16:
        r = lambda t: t.half().float()
    else:
        r = lambda t: t
    sd = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    ora = [O.pack_layer_per_head(t2n(K), t2n(V), v_bits.numpy(), k_bits.numpy(), H_Q // H_KV) for K, V in kv]
    # the module's own table: casting the model to fp16 rounded it, and prefill used it that way
    inv_freq = model.model.rotary_emb.inv_freq.detach().float().cpu()
    K_new = [np.zeros((H_KV, 0, D), np.float32) for _ in range(LAYERS)]
    V_new = [np.zeros((H_KV, 0, D), np.float32) for _ in range(LAYERS)]
    out = []
    for step, tok in enumerate(tokens):
        ang = (position0 + step) * inv_freq
        cos, sin = r(torch.cos(ang)), r(torch.sin(ang))      # the model hands out tables in its dtype

        def rope(x):       # half-split rotation, rounded to the model dtype like the in-place kernel
            lo, hi = x[:, :D // 2], x[:, D // 2:]
            return r(torch.cat([lo * cos - hi * sin, hi * cos + lo * sin], -1))

        h = sd["model.embed_tokens.weight"][tok][None]
        for i in range(LAYERS):
            p = f"model.layers.{i}."
            x = r(_rms(h, sd[p + "input_layernorm.weight"], cfg.rms_norm_eps))
            q = r(x @ sd[p + "self_attn.q_proj.weight"].T).view(H_Q, D)
            k = r(x @ sd[p + "self_attn.k_proj.weight"].T).view(H_KV, D)
            v = r(x @ sd[p + "self_attn.v_proj.weight"].T).view(H_KV, D)
            q, k = rope(q), rope(k)
            K_new[i] = np.concatenate([K_new[i], k.numpy()[:, None]], 1)
            V_new[i] = np.concatenate([V_new[i], v.numpy()[:, None]], 1)
            a = O.trizone_attention_ref(q.numpy(), ora[i][0], ora[i][1], K_new[i], V_new[i])
            a = r(torch.from_numpy(np.asarray(a, np.float32))).view(1, H_Q * D)
            h = r(h + r(a @ sd[p + "self_attn.o_proj.weight"].T))
            x = r(_rms(h, sd[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps))
            gate = r(x @ sd[p + "mlp.gate_proj.weight"].T)
            up = r(x @ sd[p + "mlp.up_proj.weight"].T)
            act = r(r(torch.nn.functional.silu(gate)) * up)
            h = r(h + r(act @ sd[p + "mlp.down_proj.weight"].T))
        h = r(_rms(h, sd["model.norm.weight"], cfg.rms_norm_eps))
        out.append((h @ sd["lm_head.weight"].T)[0])
    return out


@pytest.mark.parametrize("fp32_model", [True, False])
def test_decode_loop_matches_restated_model_over_oracle_attention(setup, fp32_model):
    """With fp32 weights and activations the only differences left are summation orders and the
    oracle's fp16 rounding of dequantized K / V: 2e-3 of the largest logit.  The fp16 model adds
    its per-operation roundings, which the restatement follows only approximately: 5e-2."""
    model, prompt, pre, kv = setup
    if fp32_model:
        import copy
        model = copy.deepcopy(model).float()
    v_bits, k_bits = _mixed_bits(11)
    cache = _pack(kv, v_bits, k_bits)
    first = pre.logits[0, -1]
    tol = 2e-3 if fp32_model else 5e-2
    ids, logits = fast_decode.greedy_decode_fast(model, cache, first, 6, [], torch.device(DEV), T_PROMPT,
                                                 return_logits=True)
    assert len(ids) == 6 and len(logits) == 6 and ids[0] == int(first.argmax())
    ref = _reference_logits(model, kv, v_bits, k_bits, ids, T_PROMPT)
    for step, (got, exp) in enumerate(zip(logits, ref)):
        got = got[0]
        scale = float(exp.abs().max())
        err = float((got - exp).abs().max())
        assert err <= tol * scale, f"step {step}: logits off by {err} (largest logit {scale})"
        if step + 1 < len(ids):
            assert ids[step + 1] == int(got.argmax())


def test_decode_loop_tracks_model_forward(setup):
    """All V kept as fp16, all K channels at 8 bits: the packed cache is the dense one up to the
    K quantization, so the loop must follow ``model.forward`` over the dense cache closely."""
    model, prompt, pre, kv = setup
    v_bits = torch.full((H_KV, T_PROMPT), 16)
    k_bits = torch.full((H_KV, D), 8)
    cache = _pack(kv, v_bits, k_bits)
    first = pre.logits[0, -1]
    ids, logits = fast_decode.greedy_decode_fast(model, cache, first, 4, [], torch.device(DEV), T_PROMPT,
                                                 return_logits=True)
    with torch.no_grad():
        again = model(prompt, use_cache=True)
        pkv = again.past_key_values
        for step, tok in enumerate(ids):
            o = model(torch.tensor([[tok]], device=DEV), past_key_values=pkv, use_cache=True)
            pkv = o.past_key_values
            exp = o.logits[0, -1].float().cpu()
            got = logits[step][0]
            cos = float(torch.nn.functional.cosine_similarity(got, exp, dim=0))
            assert cos > 0.999, f"step {step}: cosine {cos}"
            assert float((got - exp).abs().max()) <= 0.05 * float(exp.abs().max())


@pytest.mark.parametrize("n_tokens,seed", [(80, 12), (1, 3), (2, 4), (63, 5), (65, 6), (130, 7)])
def test_graph_replay_gives_the_eager_tokens(setup, n_tokens, seed):
    model, prompt, pre, kv = setup          # 80 tokens: the raw tail crosses the 64-token chunk of the merge kernel
    v_bits, k_bits = _mixed_bits(seed)
    first = pre.logits[0, -1]
    eager = fast_decode.greedy_decode_fast(model, _pack(kv, v_bits, k_bits), first, n_tokens, [], torch.device(DEV),
                                           T_PROMPT)
    cache = _pack(kv, v_bits, k_bits)
    graphed = fast_decode.greedy_decode_fast(model, cache, first, n_tokens, [], torch.device(DEV), T_PROMPT,
                                             use_cuda_graph=True)
    assert graphed == eager and len(eager) == n_tokens
    # a second run over the same cache object reuses its streaming caches and zone C buffers
    torch.cuda.synchronize()
    assert fast_decode.greedy_decode_fast(model, cache, first, n_tokens, [], torch.device(DEV), T_PROMPT,
                                          use_cuda_graph=True) == eager


def test_observers_eos_and_errors(setup):
    model, prompt, pre, kv = setup
    v_bits, k_bits = _mixed_bits(13)
    cache = _pack(kv, v_bits, k_bits)
    first = pre.logits[0, -1]
    dev = torch.device(DEV)
    ids = fast_decode.greedy_decode_fast(model, cache, first, 5, [], dev, T_PROMPT)
    seen, hid = [], []
    hidden0 = torch.zeros(1, HID, device=DEV, dtype=torch.float16)
    out = fast_decode.greedy_decode_fast(
        model, cache, first, 5, [ids[2]], dev, T_PROMPT, next_token_hidden=hidden0,
        logits_observer=lambda s, lg, t, e: seen.append((s, tuple(lg.shape), t, e)),
        hidden_observer=lambda s, hh, t, e: hid.append((s, tuple(hh.shape), t, e)))
    stop = ids.index(ids[2])           # the loop ends at the first EOS token, which is not returned
    assert out == ids[:stop]
    assert [s[0] for s in seen] == list(range(stop + 1)) and seen[-1][3] and not any(s[3] for s in seen[:-1])
    assert [s[2] for s in seen] == ids[:stop + 1]
    assert all(s[1] == (1, VOCAB) for s in seen) and all(h_[1] == (1, HID) for h_ in hid)
    with pytest.raises(NotImplementedError):
        fast_decode.greedy_decode_fast(model, cache, first, 2, [], dev, T_PROMPT, use_cuda_graph=True,
                                       return_logits=True)
    with pytest.raises(ValueError):
        fast_decode.greedy_decode_fast(model, cache, first, 2, [], dev, T_PROMPT, hidden_observer=lambda *a: None)
    W = fast_decode.pre_extract_weights(model)
    assert W is fast_decode.pre_extract_weights(model) and W.num_layers == LAYERS and W.num_kv_groups == H_Q // H_KV
    assert W.layers[0].qkv_split_sizes == (H_Q * D, H_KV * D, H_KV * D) and W.layers[0].qkv_bias is None


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_step_kernels_match_tensor_expressions(dtype):
    """The one-launch forms against the tensor expressions of fast_decode.py:628-633, 1690,
    1722-1724, 1786, 1803 (one unit in the last place where a sum is taken in another order)."""
    require_gpu()
    from rdkv_amd.triton_rope import fused_rope
    g = torch.Generator(device=DEV).manual_seed(5)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2.0 ** -22}[dtype]
    for rows, dim in ((1, 4096), (4, 128), (3, 1000), (2, 8192), (1, 16384)):
        x = torch.randn(rows, dim, generator=g, device=DEV).to(dtype)
        d = torch.randn(rows, dim, generator=g, device=DEV).to(dtype)
        w = (1.0 + 0.1 * torch.randn(dim, generator=g, device=DEV)).to(dtype)

        def expr(t):
            tf = t.float()
            return (w * (tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + 1e-5))).to(dtype)

        got = fast_decode._rms_norm(x, w, 1e-5)
        torch.testing.assert_close(got.float(), expr(x).float(), rtol=2 * ulp, atol=1e-6)
        res = x.clone()
        got = fast_decode._rms_norm(res, w, 1e-5, delta=d, residual_out=res)      # in place on the residual
        assert torch.equal(res, x + d)
        torch.testing.assert_close(got.float(), expr(x + d).float(), rtol=2 * ulp, atol=1e-6)
    gate = 3 * torch.randn(1, 1, 14336, generator=g, device=DEV).to(dtype)
    up = torch.randn(1, 1, 14336, generator=g, device=DEV).to(dtype)
    both = torch.cat([gate, up], -1)
    got = fast_decode._silu_mul(both[..., :14336], both[..., 14336:])
    exp = torch.nn.functional.silu(gate) * up
    torch.testing.assert_close(got.float(), exp.float(), rtol=2 * ulp, atol=1e-6)
    # rotate + append against the in-place rotation followed by the tensor copy
    k = torch.randn(8, 128, generator=g, device=DEV).to(dtype)
    v = torch.randn(8, 128, generator=g, device=DEV).to(dtype)
    cs = torch.rand(64, generator=g, device=DEV).to(dtype)
    sn = torch.rand(64, generator=g, device=DEV).to(dtype)
    buf = torch.full((8, 5, 256), 7.0, device=DEV)
    row = torch.tensor([3], device=DEV)
    fast_decode._rope_append_kv(k, v, cs, sn, buf, row)
    q_dummy = torch.zeros(8, 128, device=DEV, dtype=dtype)
    k_rot = k.clone()
    fused_rope(q_dummy, k_rot, cs, sn)
    assert torch.equal(buf[:, 3], torch.cat([k_rot, v], -1).float())
    assert float((buf[:, [0, 1, 2, 4]] - 7.0).abs().max()) == 0.0
    fast_decode._rope_append_kv(k, v, cs, sn, buf, torch.tensor([5], device=DEV))     # outside: nothing written
    assert float((buf[:, [0, 1, 2, 4]] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_projection_row_kernel_matches_library(dtype):
    """``_linear_row`` (one pass over the weights) against an fp64 product of the same values;
    shapes of the decode step and the edges of the row partition (N below, at and off the
    multiples of rows per wavefront; strided weight rows; bias)."""
    require_gpu()
    g = torch.Generator(device=DEV).manual_seed(9)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    for N, K, with_bias in ((6144, 4096, False), (4096, 14336, False), (28672, 4096, True), (1, 512, True),
                            (7, 512, False), (4099, 1024, True), (20000, 512, False)):
        Wfull = (torch.randn(N, K + 8, generator=g, device=DEV) / K ** 0.5).to(dtype)
        W = Wfull[:, :K]                                   # row stride K + 8
        x = torch.randn(1, 1, K, generator=g, device=DEV).to(dtype)
        b = torch.randn(N, generator=g, device=DEV).to(dtype) if with_bias else None
        got = fast_decode._linear_row(x, W, b)
        assert got.shape == (1, 1, N) and got.dtype == dtype
        exp = x.double().view(1, K) @ W.double().T + (b.double() if b is not None else 0.0)
        torch.testing.assert_close(got.double().view(1, N), exp, rtol=2 * ulp, atol=2 * ulp)
        # an fp32 row is rounded to the weights' type inside: the same bits as casting it first
        x32 = torch.randn(1, 1, K, generator=g, device=DEV)
        assert torch.equal(fast_decode._linear_row(x32, W, b), fast_decode._linear_row(x32.to(dtype), W, b))
    # shapes the kernel does not take go to the library
    W = torch.randn(16, 100, generator=g, device=DEV).to(dtype)
    x = torch.randn(1, 100, generator=g, device=DEV).to(dtype)
    torch.testing.assert_close(fast_decode._linear_row(x, W), torch.nn.functional.linear(x, W))


@pytest.mark.parametrize("family", ["qwen2", "qwen3"])
def test_decode_loop_follows_other_model_families(family):
    """q/k/v projection biases (Qwen2) and per-head q/k RMSNorm before the rotary embedding (Qwen3)
    (fast_decode.py:352-355, 381-384, 1664-1667): the loop tracks ``model.forward`` over the dense
    prompt cache when V stays fp16 and K gets 8 bits."""
    require_gpu()
    import transformers
    kw = dict(hidden_size=HID, intermediate_size=1024, num_hidden_layers=LAYERS, num_attention_heads=H_Q,
              num_key_value_heads=H_KV, vocab_size=VOCAB, max_position_embeddings=4096, tie_word_embeddings=False)
    if family == "qwen2":
        model = transformers.Qwen2ForCausalLM(transformers.Qwen2Config(**kw))
    else:
        model = transformers.Qwen3ForCausalLM(transformers.Qwen3Config(head_dim=D, **kw))
    torch.manual_seed(4321)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() == 2:
                p.copy_(torch.randn_like(p) * 0.06)
            elif name.endswith("bias"):
                p.copy_(torch.randn_like(p) * 0.5)
            else:
                p.copy_(1.0 + 0.2 * torch.randn_like(p))       # norm weights, q_norm / k_norm included
    model = model.half().to(DEV).eval()
    W = fast_decode.pre_extract_weights(model)
    assert (W.layers[0].qkv_bias is not None) == (family == "qwen2")
    assert (W.layers[0].q_norm_weight is not None) == (family == "qwen3")
    g = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, VOCAB, (1, 200), generator=g).to(DEV)
    with torch.no_grad():
        pre = model(prompt, use_cache=True)
        kv = [(l.keys.contiguous(), l.values.contiguous()) for l in pre.past_key_values.layers[:LAYERS]]
    layers, v16 = [], []
    for K, V in kv:
        pl, nvo = packing.pack_layer_per_head(K, V, torch.full((H_KV, 200), 16), torch.full((H_KV, D), 8), H_Q // H_KV)
        layers.append(pl)
        v16.append(nvo)
    cache = packing.TriZoneCache(tuple(layers), v16, [None] * LAYERS, [None] * LAYERS, 200)
    ids, logits = fast_decode.greedy_decode_fast(model, cache, pre.logits[0, -1], 4, [], torch.device(DEV), 200,
                                                 return_logits=True)
    with torch.no_grad():
        pkv = model(prompt, use_cache=True).past_key_values
        for step, tok in enumerate(ids):
            o = model(torch.tensor([[tok]], device=DEV), past_key_values=pkv, use_cache=True)
            pkv = o.past_key_values
            exp, got = o.logits[0, -1].float().cpu(), logits[step][0]
            cos = float(torch.nn.functional.cosine_similarity(got, exp, dim=0))
            assert cos > 0.999, f"{family} step {step}: cosine {cos}"
    assert fast_decode.greedy_decode_fast(model, cache, pre.logits[0, -1], 4, [], torch.device(DEV), 200,
                                          use_cuda_graph=True) == ids


def test_graph_replay_with_model_sized_projections():
    """Llama-3.1-8B-sized projections and vocabulary (two layers): every token of 70 graph replays
    equals the eager run's - the argmax over 128 256 logits, the large GEMVs and the merge with a
    raw tail past one chunk all sit inside the captured step."""
    require_gpu()
    from transformers import LlamaConfig, LlamaForCausalLM
    from rdkv_amd import synth
    L = 2
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=L, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=8192,
                      rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False)
    torch.manual_seed(0)
    with torch.device(DEV):
        model = LlamaForCausalLM(cfg).half().eval()
    sc = synth.scaled(synth.CONFIGS[1], layers=L, context=1024)
    layers, v16 = [], []
    for i in range(L):
        vb, kb, oc = synth.layer_allocation(sc, i)
        K, V, _ = synth.layer_data(sc, i, DEV, outliers=oc)
        pl, nvo = packing.pack_layer_per_head(K, V, vb, kb, sc.G)
        layers.append(pl)
        v16.append(nvo)
    cache = packing.TriZoneCache(tuple(layers), v16, [None] * L, [None] * L, sc.context)
    first = torch.randn(cfg.vocab_size, generator=torch.Generator().manual_seed(1)).to(DEV)
    dev = torch.device(DEV)
    eager = fast_decode.greedy_decode_fast(model, cache, first, 70, [], dev, sc.context)
    graphed = fast_decode.greedy_decode_fast(model, cache, first, 70, [], dev, sc.context, use_cuda_graph=True)
    assert graphed == eager and len(set(eager)) > 35
    del model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_row_projections_match_their_compositions(dtype):
    """``_norm_linear_row`` (residual add + RMSNorm folded into the GEMV's staging) and
    ``_silu_linear_row`` against the separate launches they replace; shapes the fused kernels do
    not take fall back to those launches."""
    require_gpu()
    g = torch.Generator(device=DEV).manual_seed(21)
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    for N, K in ((6144, 4096), (1000, 512), (28672, 4096), (300, 8192)):
        W = (torch.randn(N, K, generator=g, device=DEV) / K ** 0.5).to(dtype)
        h = torch.randn(1, 1, K, generator=g, device=DEV).to(dtype)
        d = torch.randn(1, 1, K, generator=g, device=DEV).to(dtype)
        nw = (1.0 + 0.1 * torch.randn(K, generator=g, device=DEV)).to(dtype)
        b = torch.randn(N, generator=g, device=DEV).to(dtype)
        for delta, bias in ((d, None), (None, b), (d, b)):
            h_in = h.clone()
            y, h_new = fast_decode._norm_linear_row(h_in, delta, nw, 1e-5, W, bias)
            assert torch.equal(h_in, h), "the fused form leaves its inputs alone"
            exp_h = h + delta if delta is not None else h
            assert torch.equal(h_new, exp_h)
            x = fast_decode._rms_norm(exp_h, nw, 1e-5)
            exp = x.double().view(1, K) @ W.double().T + (bias.double() if bias is not None else 0.0)
            torch.testing.assert_close(y.double().view(1, N), exp, rtol=4 * ulp, atol=4 * ulp)
    for N, K in ((4096, 14336), (512, 1024)):
        W = (torch.randn(N, K, generator=g, device=DEV) / K ** 0.5).to(dtype)
        gu = (2 * torch.randn(1, 1, 2 * K, generator=g, device=DEV)).to(dtype)
        gate, up = gu.split((K, K), dim=-1)
        assert torch.equal(fast_decode._silu_linear_row(gate, up, W),
                           fast_decode._linear_row(fast_decode._silu_mul(gate, up), W))
    # K outside the fused kernels: the separate launches
    W = torch.randn(32, 16384, generator=g, device=DEV).to(dtype) * 0.01
    h = torch.randn(1, 1, 16384, generator=g, device=DEV).to(dtype)
    nw = torch.ones(16384, device=DEV, dtype=dtype)
    y, h2 = fast_decode._norm_linear_row(h, None, nw, 1e-5, W)
    torch.testing.assert_close(y, fast_decode._linear_row(fast_decode._rms_norm(h, nw, 1e-5), W))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_argmax_and_advance_matches_the_library_argmax(dtype):
    """`rdkv_argmax_advance`: the index `argmax` returns (first of equal maxima, a NaN before any
    number) for vocabulary sizes with and without a ragged end, and the step's counters moved on."""
    g = torch.Generator().manual_seed(11)
    for n in (128256, 151936, 8193, 1000, 9, 7, 1):
        x = torch.randn(n, generator=g) * 3
        cases = [x.clone()]
        if n > 8:
            tie = x.clone()
            tie[[n - 1, n // 2, 5]] = 50.0                      # equal maxima: the lowest index wins
            nan = x.clone()
            nan[[n - 2, 3]] = float("nan")                       # a NaN counts as the maximum
            low = torch.full((n,), -float("inf"))
            last = x.clone()
            last[n - 1] = 60.0                                    # the maximum in the ragged end
            cases += [tie, nan, low, last]
        for c in cases:
            logits = c.to(dtype).to(DEV).view(1, 1, n)
            token = torch.full((1, 1), -1, dtype=torch.long, device=DEV)
            pos = torch.tensor([[41]], dtype=torch.long, device=DEV)
            row = torch.tensor([6], dtype=torch.long, device=DEV)
            counts = torch.tensor([3, 9, 1], dtype=torch.int32, device=DEV)
            fast_decode._argmax_advance(logits, token, pos, row, counts)
            assert int(token) == int(torch.argmax(c.to(dtype).float())), (n, dtype)
            assert int(pos) == 42 and int(row) == 7 and counts.tolist() == [4, 10, 2]
