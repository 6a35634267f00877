"""The blockwise decode loop (``blockwise_decode.greedy_decode_blockwise``) on a small
random-weight Llama: schedule, report and coverage as the reference defines them
(blockwise_decode.py:1124-2260), tokens / logits against ``model.forward`` when the blocks keep
full precision, and the bounds the online block scores obey as sums of softmax weights."""
import pytest
import torch

from rdkv_amd import blockwise_decode as bw
from rdkv_amd import fast_decode, knapsack_solver as ks, packing
from tests.gpu_util import DEV, require_gpu

pytestmark = pytest.mark.gpu

T_PROMPT, H_Q, H_KV, D, HID, LAYERS, VOCAB = 160, 4, 2, 128, 512, 2, 1000


@pytest.fixture(scope="module")
def setup():
    require_gpu()
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(hidden_size=HID, intermediate_size=1024, num_hidden_layers=LAYERS, num_attention_heads=H_Q,
                      num_key_value_heads=H_KV, head_dim=D, vocab_size=VOCAB, max_position_embeddings=4096,
                      rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False)
    torch.manual_seed(99)
    model = LlamaForCausalLM(cfg)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 2:
                p.mul_(3.0)
    model = model.half().to(DEV).eval()
    g = torch.Generator().manual_seed(8)
    prompt = torch.randint(0, VOCAB, (1, T_PROMPT), generator=g).to(DEV)
    with torch.no_grad():
        pre = model(prompt, use_cache=True)
    layers, v16 = [], []
    for i in range(LAYERS):
        l = pre.past_key_values.layers[i]
        pl, nvo = packing.pack_layer_per_head(l.keys.contiguous(), l.values.contiguous(),
                                              torch.full((H_KV, T_PROMPT), 16), torch.full((H_KV, D), 8), H_Q // H_KV)
        layers.append(pl)
        v16.append(nvo)
    cache = packing.TriZoneCache(tuple(layers), v16, [None] * LAYERS, [None] * LAYERS, T_PROMPT)
    return model, prompt, pre, cache


def _config(block, budget):
    return bw.BlockwiseRDKVConfig(block_size=block, block_budget_tokens=budget, k_budget_ratio=0.5, obs_window=4,
                                  pool_kernel_size=3, pool_padding="reflect",
                                  v_bit_options=torch.tensor([0., 2, 4, 8, 16]),
                                  k_bit_options=torch.tensor([0., 2, 4, 8]),
                                  epsilon_v=ks.DEFAULT_EPSILON_V, epsilon_k=ks.DEFAULT_EPSILON_K,
                                  correctness_check=True)


@pytest.mark.parametrize("n_tokens", [37, 48, 5])
def test_schedule_report_and_coverage(setup, n_tokens):
    model, prompt, pre, cache = setup
    block = 16
    ids, report = bw.greedy_decode_blockwise(
        model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1], max_new_tokens=n_tokens,
        eos_token_ids=[], primary_device=torch.device(DEV), decode_position_start=T_PROMPT, config=_config(block, 4))
    assert len(ids) == n_tokens and report["generated_tokens"] == n_tokens
    plan = bw.plan_block_compressions(n_tokens, block)
    assert report["num_compressed_decode_blocks"] == len(plan) == len(report["block_events"])
    cov = report["coverage"]
    assert cov[0][0] == 0 and cov[-1][1] == n_tokens - 1
    assert all(a[1] + 1 == b[0] for a, b in zip(cov, cov[1:]))
    for ev, exp in zip(report["block_events"], plan):
        assert all(ev[k] == exp[k] for k in exp)
    assert len(report["per_token_timestamps_ms"]) == n_tokens
    assert report["decode_cache_peak_fp16_equivalent_tokens"] <= 2 * block + 4 * len(plan) + 1e-6
    assert report["memory_trace"][0]["stage"] == "decode_start" and report["memory_trace"][-1]["stage"] == "decode_complete"
    assert report["avg_tpot_ms"] > 0 and report["decode_cuda_graph"] is False
    # the prompt's own per-layer caches are untouched: the plain loop still runs on them
    again = fast_decode.greedy_decode_fast(model, cache, pre.logits[0, -1], 3, [], torch.device(DEV), T_PROMPT)
    assert again == ids[:3]


def test_full_precision_blocks_track_model_forward(setup):
    """Budget = block size: every block keeps 16-bit V and 8-bit K, so the loop over
    [prompt | blocks | tail] must follow ``model.forward`` over the dense cache."""
    model, prompt, pre, cache = setup
    n_tokens, block = 30, 8
    seen = []
    orig = fast_decode._linear_row

    def spy(x, weight, bias=None):
        y = orig(x, weight, bias)
        if weight is model.lm_head.weight:
            seen.append(y[0, -1].float().cpu())
        return y

    fast_decode._linear_row = spy
    try:
        ids, report = bw.greedy_decode_blockwise(
            model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1], max_new_tokens=n_tokens,
            eos_token_ids=[], primary_device=torch.device(DEV), decode_position_start=T_PROMPT,
            config=_config(block, block))
    finally:
        fast_decode._linear_row = orig
    assert report["num_compressed_decode_blocks"] == 4 and len(seen) == n_tokens
    with torch.no_grad():
        pkv = model(prompt, use_cache=True).past_key_values
        for step, tok in enumerate(ids):
            o = model(torch.tensor([[tok]], device=DEV), past_key_values=pkv, use_cache=True)
            pkv = o.past_key_values
            exp = o.logits[0, -1].float().cpu()
            cos = float(torch.nn.functional.cosine_similarity(seen[step], exp, dim=0))
            assert cos > 0.998, f"step {step}: cosine {cos}"


def test_block_scores_are_sums_of_softmax_weights(setup, monkeypatch):
    """What ``_compress_block`` receives: per layer [H_kv, block tokens] scores that are sums, over
    the scoring queries and the group's heads, of softmax weights (blockwise_decode.py:2085-2109):
    non-negative, and a token cannot collect more than one unit per (query, head)."""
    model, prompt, pre, cache = setup
    block, n_tokens, G = 8, 29, H_Q // H_KV
    calls = []
    orig = bw._compress_block

    def spy(**kw):
        calls.append({k: kw[k] for k in ("token_scores_by_layer", "query_block", "causal", "token_start", "token_end")})
        return orig(**kw)

    monkeypatch.setattr(bw, "_compress_block", spy)
    bw.greedy_decode_blockwise(model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1],
                               max_new_tokens=n_tokens, eos_token_ids=[], primary_device=torch.device(DEV),
                               decode_position_start=T_PROMPT, config=_config(block, 3))
    assert len(calls) == 4
    for c in calls:
        n_target = c["token_end"] - c["token_start"] + 1
        n_query = c["query_block"][0].shape[1]
        for scores, queries in zip(c["token_scores_by_layer"], c["query_block"]):
            assert tuple(scores.shape) == (H_KV, n_target) and tuple(queries.shape) == (H_Q, n_query, D)
            assert torch.isfinite(scores).all() and float(scores.min()) >= 0.0
            assert float(scores.max()) <= G * n_query + 1e-4
            assert float(scores.sum(dim=1).max()) <= G * n_query + 1e-4
            if c["causal"]:       # every query attends at least to itself: the diagonal mass is positive
                assert float(scores.sum()) > 0.0


def test_eos_stops_and_flushes(setup):
    model, prompt, pre, cache = setup
    ids, _ = bw.greedy_decode_blockwise(
        model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1], max_new_tokens=20, eos_token_ids=[],
        primary_device=torch.device(DEV), decode_position_start=T_PROMPT, config=_config(8, 2))
    out, report = bw.greedy_decode_blockwise(
        model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1], max_new_tokens=20,
        eos_token_ids=[ids[11]], primary_device=torch.device(DEV), decode_position_start=T_PROMPT,
        config=_config(8, 2))
    stop = ids.index(ids[11])
    assert out == ids[:stop] and report["generated_tokens"] == stop
    assert report["coverage"][-1][1] == stop - 1 if stop else report["coverage"] == []
    with pytest.raises(RuntimeError):
        bw.greedy_decode_blockwise(model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1],
                                   max_new_tokens=4, eos_token_ids=[], primary_device=torch.device("cpu"),
                                   decode_position_start=T_PROMPT, config=_config(8, 2))


def test_tail_scores_kernel_matches_tensor_expressions():
    """``rdkv_tail_scores`` against blockwise_decode.py:2085-2109 of the reference as tensor
    operations, for a query in the first and in the second block of the tail."""
    require_gpu()
    from rdkv_amd import _lib
    lib = _lib.load()
    h_kv, G, block = 3, 4, 16
    g = torch.Generator(device=DEV).manual_seed(6)
    for write_pos in (0, 5, 15, 16, 23, 31):
        current_len = write_pos + 1
        qbs = (write_pos // block) * block
        w = torch.rand(h_kv * G, 2 * block + 3, generator=g, device=DEV)
        self_s = torch.rand(h_kv, 2 * block, generator=g, device=DEV)
        next_s = torch.rand(h_kv, block, generator=g, device=DEV)
        exp_self, exp_next = self_s.clone(), next_s.clone()
        exp_self[:, qbs:current_len] += w[:, qbs:current_len].view(h_kv, G, current_len - qbs).sum(dim=1)
        if qbs >= block:
            exp_next += w[:, :block].view(h_kv, G, block).sum(dim=1)
        _lib.check(lib.rdkv_tail_scores(w.data_ptr(), w.stride(0), h_kv, G, qbs, current_len, block,
                                        self_s.data_ptr(), self_s.stride(0), next_s.data_ptr(), next_s.stride(0),
                                        _lib.stream_of(torch.device(DEV))))
        torch.testing.assert_close(self_s, exp_self, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(next_s, exp_next, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("n_tokens,block", [(45, 8), (16, 8), (3, 8), (70, 16), (1, 8), (8, 8), (9, 8), (33, 4), (64, 32),
                                            (17, 16)])
def test_graph_replayed_loop_equals_the_eager_loop(setup, n_tokens, block):
    """``use_cuda_graph=True`` (blockwise_decode.py:1991-2117): the step replayed from a HIP graph,
    recorded again after every compression, gives the eager loop's tokens, compression events and
    report - through several compressions, for a run that ends on a block boundary, one shorter
    than the first graph, and with an EOS in the middle; and again on a second run over the same
    prompt cache."""
    model, prompt, pre, cache = setup
    common = dict(model=model, dual_cache=cache, next_token_logits=pre.logits[0, -1], max_new_tokens=n_tokens,
                  primary_device=torch.device(DEV), decode_position_start=T_PROMPT, config=_config(block, 4))
    ids_e, rep_e = bw.greedy_decode_blockwise(eos_token_ids=[], **common)
    for run in range(2):
        ids_g, rep_g = bw.greedy_decode_blockwise(eos_token_ids=[], use_cuda_graph=True, **common)
        assert ids_g == ids_e, f"run {run}: tokens differ"
        assert rep_g["decode_cuda_graph"] is True and rep_e["decode_cuda_graph"] is False
        assert rep_g["coverage"] == rep_e["coverage"]
        for eg, ee in zip(rep_g["block_events"], rep_e["block_events"]):
            for key in ("block_id", "token_start", "token_end", "query_source_block", "is_final_flush", "query_mode",
                        "logical_allocated_bits_per_layer", "v_bit_histogram", "k_bit_histogram", "physical_bytes"):
                assert eg[key] == ee[key], (key, eg[key], ee[key])
        assert len(rep_g["per_token_timestamps_ms"]) == len(ids_g)
    if len(ids_e) > 6:
        eos = ids_e[len(ids_e) // 2]
        stop = ids_e.index(eos)
        ids_s, rep_s = bw.greedy_decode_blockwise(eos_token_ids=[eos], use_cuda_graph=True, **common)
        assert ids_s == ids_e[:stop] and rep_s["generated_tokens"] == stop
