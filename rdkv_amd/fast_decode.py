"""Attention section of the reference's decode loop (obkv_accel/fast_decode.py:1701-1784) on
the HIP kernels, plus the host-side helpers that section relies on.

Three zones per layer: A = compressed prompt tokens (packed K + packed V), B = prompt tokens
whose V stays fp16 (packed K + ``new_v_only``), C = tokens appended during decode (fp32 K|V in
``new_kv_buf``).  ``trizone_attention`` follows the reference's sequence of calls on the
padded layout; ``trizone_attention_fused`` does zones A+B in the fused streaming kernel and
merges zone C exactly through the log-sum-exp.

``greedy_decode_fast`` is the reference's decode loop around that section for a Llama-style
model on one GPU: projections, MLP and LM head are library GEMVs (plumbing), attention is the
fused streaming kernel, and with ``use_cuda_graph`` the whole step is one HIP graph.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from .k_kernel import INV_SQRT_D, k_mixed_qk_dot_into
from .packing import PackedKVLayer
from .stream_cache import StreamCache, build_stream_cache, decode_attn_fused
from .v_kernel import v_dequant_weighted_sum_dispatch_into


def _rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, *, delta: Optional[torch.Tensor] = None,
              residual_out: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of the decode loop (fast_decode.py:628-633): ``weight * (x.float() * rsqrt(mean(x^2) +
    eps))`` rounded to ``x.dtype``, one launch (``rdkv_add_rms_norm``).  ``delta``: the residual
    branch to add first (``x + delta`` rounded to the dtype, as the tensor add stores it);
    ``residual_out`` (may be ``x``) receives that sum."""
    dev = _lib.require_device(x, weight)
    dim = x.shape[-1]
    assert x.dtype in _lib.DTYPE_CODE and weight.dtype in _lib.DTYPE_CODE and weight.numel() == dim
    x2 = x.reshape(-1, dim)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=dev)
    o2 = out.view(-1, dim)
    d2 = r2 = None
    if delta is not None:
        assert delta.dtype == x.dtype and delta.numel() == x.numel()
        d2 = delta.reshape(-1, dim)
        if d2.stride(1) != 1:
            d2 = d2.contiguous()
    if residual_out is not None:
        assert residual_out.dtype == x.dtype and residual_out.numel() == x.numel() and residual_out.is_contiguous()
        r2 = residual_out.view(-1, dim)
    w = weight if weight.is_contiguous() else weight.contiguous()
    _lib.check(_lib.load().rdkv_add_rms_norm(
        x2.data_ptr(), x2.stride(0), _lib.ptr(d2), d2.stride(0) if d2 is not None else 0, w.data_ptr(),
        _lib.DTYPE_CODE[w.dtype], float(eps), rows, dim, _lib.DTYPE_CODE[x.dtype], _lib.ptr(r2),
        r2.stride(0) if r2 is not None else 0, o2.data_ptr(), o2.stride(0), _lib.stream_of(dev)))
    return out


def _rope_append_kv(k_2d: torch.Tensor, v_2d: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor,
                    new_kv_rows: torch.Tensor, row: torch.Tensor) -> None:
    """Rotate the new token's k and store fp32 [k | v] as row ``row[0]`` (device int64) of the zone C
    buffer ``new_kv_rows`` [H_kv, capacity, 2*D] (fast_decode.py:1690, 1722-1724) in one launch."""
    dev = _lib.require_device(k_2d, v_2d, cos_half, sin_half, new_kv_rows, row)
    H_kv, D = k_2d.shape
    assert v_2d.shape == (H_kv, D) and k_2d.dtype == v_2d.dtype and k_2d.dtype in _lib.DTYPE_CODE
    assert k_2d.stride(1) == 1 and v_2d.stride(1) == 1
    assert new_kv_rows.dtype == torch.float32 and new_kv_rows.shape[0] == H_kv and new_kv_rows.shape[2] == 2 * D
    assert new_kv_rows.stride(2) == 1 and row.dtype == torch.int64 and row.numel() == 1
    assert cos_half.numel() == D // 2 and sin_half.numel() == D // 2 and cos_half.dtype == sin_half.dtype
    cos_half, sin_half = cos_half.contiguous(), sin_half.contiguous()
    _lib.check(_lib.load().rdkv_rope_append_kv(
        k_2d.data_ptr(), k_2d.stride(0), v_2d.data_ptr(), v_2d.stride(0), H_kv, D, _lib.DTYPE_CODE[k_2d.dtype],
        cos_half.data_ptr(), sin_half.data_ptr(), _lib.DTYPE_CODE[cos_half.dtype], new_kv_rows.data_ptr(),
        new_kv_rows.stride(0), new_kv_rows.stride(1), row.data_ptr(), new_kv_rows.shape[1], _lib.stream_of(dev)))


def _argmax_advance(logits: torch.Tensor, token: torch.Tensor, position: Optional[torch.Tensor] = None,
                    write_row: Optional[torch.Tensor] = None, n_new: Optional[torch.Tensor] = None) -> None:
    """``token <- argmax(logits)`` (fast_decode.py:1827) and, where given, ``position``, ``write_row``
    (int64, one element each) and every ``n_new`` (int32) advanced by one, in one launch instead of
    the reduction's two and four elementwise ones."""
    dev = _lib.require_device(logits, token, *(t for t in (position, write_row, n_new) if t is not None))
    row = logits.reshape(-1)
    assert row.is_contiguous() and row.dtype in _lib.DTYPE_CODE and row.data_ptr() % 16 == 0
    assert token.dtype == torch.int64 and token.numel() == 1
    for t in (position, write_row):
        assert t is None or (t.dtype == torch.int64 and t.numel() == 1)
    assert n_new is None or (n_new.dtype == torch.int32 and n_new.is_contiguous() and n_new.numel() <= 1024)
    _lib.check(_lib.load().rdkv_argmax_advance(row.data_ptr(), row.numel(), _lib.DTYPE_CODE[row.dtype],
                                               token.data_ptr(), _lib.ptr(position), _lib.ptr(write_row),
                                               _lib.ptr(n_new), 0 if n_new is None else n_new.numel(),
                                               _lib.stream_of(dev)))


def _linear_row(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``F.linear(x.to(weight.dtype), weight, bias)`` for the single activation row of a decode
    step (fast_decode.py:1650-1656, 1785-1786, 1797-1804, 1826): one pass over the weights with
    ``rdkv_gemv`` when the shape allows it (fp16 / bf16 weights, K a multiple of 512 up to 32768,
    16-byte aligned rows; x of the weights' type or fp32, which the kernel rounds while staging
    it), the library GEMM otherwise."""
    dev = _lib.require_device(x, weight)          # no CPU path: the library product below is the GPU's too
    N, K = weight.shape
    ok = (x.numel() == K and x.dtype in (weight.dtype, torch.float32)
          and weight.dtype in (torch.float16, torch.bfloat16)
          and K % 512 == 0 and K <= 32768 and weight.stride(1) == 1 and weight.stride(0) % 8 == 0
          and weight.data_ptr() % 16 == 0 and x.is_contiguous() and x.data_ptr() % 16 == 0
          and (bias is None or (bias.dtype == weight.dtype and bias.is_contiguous())))
    if not ok:
        return F.linear(x.to(weight.dtype), weight, bias)
    y = torch.empty(x.shape[:-1] + (N,), dtype=weight.dtype, device=dev)
    _lib.check(_lib.load().rdkv_gemv(weight.data_ptr(), weight.stride(0), x.data_ptr(), _lib.DTYPE_CODE[x.dtype],
                                     _lib.ptr(bias), N, K, _lib.DTYPE_CODE[weight.dtype], y.data_ptr(),
                                     _lib.stream_of(dev)))
    return y


def _row_ok(*tensors: torch.Tensor) -> bool:
    return all(t.is_contiguous() and t.data_ptr() % 16 == 0 for t in tensors)


def _gemv_weight_ok(weight: torch.Tensor, bias: Optional[torch.Tensor], k_max: int) -> bool:
    K = weight.shape[1]
    return (weight.dtype in (torch.float16, torch.bfloat16) and K % 512 == 0 and K <= k_max
            and weight.stride(1) == 1 and weight.stride(0) % 8 == 0 and weight.data_ptr() % 16 == 0
            and (bias is None or (bias.dtype == weight.dtype and bias.is_contiguous())))


def _norm_linear_row(h: torch.Tensor, delta: Optional[torch.Tensor], norm_weight: torch.Tensor, eps: float,
                     weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Residual add, RMSNorm and projection of one activation row (fast_decode.py:1640-1656 and
    1786-1798): returns ``(F.linear(rms_norm(h + delta), weight, bias), h + delta)``.  One launch
    (``rdkv_gemv_norm``: the norm is folded into the staging of the row) when the shapes allow it,
    ``_rms_norm`` + ``_linear_row`` otherwise."""
    dev = _lib.require_device(h, weight)
    N, K = weight.shape
    fused = (_gemv_weight_ok(weight, bias, 8192) and h.numel() == K and h.dtype == weight.dtype
             and norm_weight.dtype == weight.dtype and _row_ok(h, norm_weight)
             and (delta is None or (delta.dtype == h.dtype and delta.numel() == K and _row_ok(delta))))
    if not fused:
        x = _rms_norm(h, norm_weight, eps, delta=delta, residual_out=h)
        return _linear_row(x, weight, bias), h
    h_new = torch.empty_like(h) if delta is not None else h
    y = torch.empty(h.shape[:-1] + (N,), dtype=weight.dtype, device=dev)
    _lib.check(_lib.load().rdkv_gemv_norm(
        weight.data_ptr(), weight.stride(0), h.data_ptr(), _lib.ptr(delta), norm_weight.data_ptr(), float(eps),
        h_new.data_ptr() if delta is not None else None, _lib.ptr(bias), N, K, _lib.DTYPE_CODE[weight.dtype],
        y.data_ptr(), _lib.stream_of(dev)))
    return y, h_new


def _silu_linear_row(gate: torch.Tensor, up: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``F.linear(F.silu(gate) * up, weight)`` for one row (fast_decode.py:1803-1804): one launch
    (``rdkv_gemv_silu``) when the shapes allow it, ``_silu_mul`` + ``_linear_row`` otherwise."""
    dev = _lib.require_device(gate, up, weight)
    N, K = weight.shape
    fused = (_gemv_weight_ok(weight, None, 32768) and gate.numel() == K and up.numel() == K
             and gate.dtype == weight.dtype and up.dtype == weight.dtype and gate.stride(-1) == 1
             and up.stride(-1) == 1 and gate.data_ptr() % 16 == 0 and up.data_ptr() % 16 == 0)
    if not fused:
        return _linear_row(_silu_mul(gate, up), weight)
    y = torch.empty(gate.shape[:-1] + (N,), dtype=weight.dtype, device=dev)
    _lib.check(_lib.load().rdkv_gemv_silu(weight.data_ptr(), weight.stride(0), gate.data_ptr(), up.data_ptr(), None,
                                          N, K, _lib.DTYPE_CODE[weight.dtype], y.data_ptr(), _lib.stream_of(dev)))
    return y


def _silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``F.silu(gate) * up`` (fast_decode.py:1803) in one launch; both [..., n] with unit stride."""
    dev = _lib.require_device(gate, up)
    assert gate.shape == up.shape and gate.dtype == up.dtype and gate.dtype in _lib.DTYPE_CODE
    n = gate.numel()
    assert gate.shape[-1] == n and gate.stride(-1) == 1 and up.stride(-1) == 1, "one row of gate / up values"
    out = torch.empty(gate.shape, dtype=gate.dtype, device=dev)
    _lib.check(_lib.load().rdkv_silu_mul(gate.data_ptr(), up.data_ptr(), n, _lib.DTYPE_CODE[gate.dtype],
                                         out.data_ptr(), _lib.stream_of(dev)))
    return out


_SQUEEZE_FIELDS = ("K_2bit", "K_4bit", "K_8bit", "K_ch_scale", "K_ch_zp", "V_2bit", "V_4bit", "V_8bit",
                   "V_scale", "V_zp")


def _pre_squeeze_packed(packed_layers: Tuple[PackedKVLayer, ...]) -> List[PackedKVLayer]:
    """Drop the leading batch dim of every kernel-consumed tensor once per cache
    (fast_decode.py:637-681).  Metadata fields are carried over; the transient
    ``deferred_k_for_stack`` is not."""
    import dataclasses
    out = []
    for pl in packed_layers:
        kw = {f.name: getattr(pl, f.name) for f in dataclasses.fields(pl)}
        for name in _SQUEEZE_FIELDS:
            if kw[name] is not None:
                kw[name] = kw[name].squeeze(0)
        kw["deferred_k_for_stack"] = None
        out.append(PackedKVLayer(**kw))
    return out


def trizone_attention(q_2d: torch.Tensor, sp: PackedKVLayer, V16: Optional[torch.Tensor],
                      n_v16_per_head: Optional[torch.Tensor], K_new: torch.Tensor, V_new: torch.Tensor,
                      num_kv_groups: int, *, scores_buf: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One layer's decode attention over zones A, B, C (fast_decode.py:1707-1784).

    q_2d [H_q,128] (rotated); sp a packed layer (4-D or pre-squeezed); V16 [H_kv,max_n_v16,128]
    fp16 or None; K_new / V_new [H_kv, n_new, 128] fp32 including the current token (n_new >= 1).
    Returns fp32 [H_q,128].  ``scores_buf`` [H_q, >= T_old + n_new] fp32 and ``out`` may be
    passed to avoid allocations (e.g. under graph capture)."""
    dev = _lib.require_device(q_2d, K_new, V_new)
    lib = _lib.load()
    H_q, D = q_2d.shape
    H_kv = H_q // num_kv_groups
    n_new = K_new.shape[1]
    T_v = int(sp.T_eff)
    T_old = int(sp.T_eff_k) if sp.T_eff_k > 0 else T_v
    if scores_buf is None:
        scores_buf = torch.empty(H_q, T_old + n_new, dtype=torch.float32, device=dev)
    if out is None:
        out = torch.empty(H_q, D, dtype=torch.float32, device=dev)
    q32 = q_2d.float()
    s_old = scores_buf[:, :T_old]
    s_new = scores_buf[:, T_old:T_old + n_new]
    if T_old > 0:
        k_mixed_qk_dot_into(q32, sp, T_old, s_old)
    # zone C scores: fp32 bmm of the scaled query group with the appended keys (:1730-1733)
    q_gqa = q32.view(H_kv, num_kv_groups, D) * INV_SQRT_D
    s_new.copy_(torch.bmm(q_gqa, K_new.transpose(-1, -2)).reshape(H_q, n_new))
    # mask + global softmax over [A | B | C], written back in place as weights (:1743-1755)
    mask = sp.softmax_mask if (T_old > 0 and sp.softmax_mask is not None) else None
    ws = _lib.workspace(dev, lib.rdkv_softmax_rows_workspace_bytes(H_q))
    _lib.check(lib.rdkv_softmax_rows_ws(
        _lib.ptr(s_old), scores_buf.stride(0), _lib.ptr(mask), mask.stride(0) if mask is not None else 0,
        T_old, s_new.data_ptr(), scores_buf.stride(0), n_new,
        _lib.ptr(s_old), scores_buf.stride(0), s_new.data_ptr(), scores_buf.stride(0), H_q,
        ws.data_ptr(), ws.numel(), _lib.stream_of(dev)))
    if T_old > 0:
        v_dequant_weighted_sum_dispatch_into(s_old, sp, out, V16=V16, n_v16_per_head=n_v16_per_head,
                                             max_T_v=T_v)
    else:
        out.zero_()
    # zone C values (:1780-1784)
    out.add_(torch.bmm(s_new.reshape(H_kv, num_kv_groups, n_new), V_new).reshape(H_q, D))
    return out


def merge_zone_c(out_ab: torch.Tensor, lse_ab: torch.Tensor, q_2d: torch.Tensor, K_new: torch.Tensor,
                 V_new: torch.Tensor, num_kv_groups: int) -> torch.Tensor:
    """Exact merge of the fused kernel's zones A+B result with the fp32 zone C attention.

    softmax over the union = weights proportional to exp(lse_ab) for the A+B block and
    exp(score) for every zone-C token.  A layer without prompt tokens has lse_ab = -inf and
    contributes nothing (never forms -inf - -inf)."""
    H_q, D = q_2d.shape
    H_kv = H_q // num_kv_groups
    if K_new.shape[-2] == 0:      # nothing appended yet: zones A+B are the whole context
        return out_ab.clone()
    q_gqa = q_2d.float().view(H_kv, num_kv_groups, D) * INV_SQRT_D
    s_new = torch.bmm(q_gqa, K_new.transpose(-1, -2)).reshape(H_q, -1)
    m = torch.maximum(lse_ab, s_new.max(dim=-1).values)
    w_ab = torch.exp(lse_ab - m)
    w_new = torch.exp(s_new - m[:, None])
    denom = w_ab + w_new.sum(-1)
    out_new = torch.bmm(w_new.view(H_kv, num_kv_groups, -1), V_new).reshape(H_q, D)
    return (out_ab * w_ab[:, None] + out_new) / denom[:, None]


def trizone_attention_fused(cache: StreamCache, q_all: torch.Tensor, K_new: List[torch.Tensor],
                            V_new: List[torch.Tensor], num_kv_groups: int, *, rope=None,
                            merge_on_host: bool = False) -> torch.Tensor:
    """All three zones of every layer / sequence of ``cache`` in two launches: the fused kernel
    over zones A+B, then a merge launch that also attends over the decode-appended tokens
    (zone C) and returns the softmax over the union.  q_all [groups*H_q,128]; K_new[g],
    V_new[g] [H_kv,n_new_g,128] fp32.  ``merge_on_host`` keeps the zone C merge as PyTorch
    operations per group (``merge_zone_c``), the cross-check of the fused merge."""
    if merge_on_host:
        assert rope is None
        out, lse = decode_attn_fused(cache, q_all)
        H_q = cache.rows // len(K_new)
        res = torch.empty_like(out)
        for g, (kn, vn) in enumerate(zip(K_new, V_new)):
            r = slice(g * H_q, (g + 1) * H_q)
            res[r] = merge_zone_c(out[r], lse[r], q_all[r], kn, vn, num_kv_groups)
        return res
    n_max = max(int(k.shape[1]) for k in K_new)
    H_kv = int(K_new[0].shape[0])
    dev = q_all.device
    if all(int(k.shape[1]) == n_max for k in K_new):
        kn = torch.stack([k.float() for k in K_new]).reshape(-1, n_max, 128)
        vn = torch.stack([v.float() for v in V_new]).reshape(-1, n_max, 128)
        counts = None
    else:
        kn = torch.zeros(len(K_new) * H_kv, n_max, 128, dtype=torch.float32, device=dev)
        vn = torch.zeros_like(kn)
        for g, (k, v) in enumerate(zip(K_new, V_new)):
            kn[g * H_kv:(g + 1) * H_kv, :k.shape[1]] = k
            vn[g * H_kv:(g + 1) * H_kv, :v.shape[1]] = v
        counts = torch.tensor([int(k.shape[1]) for k in K_new for _ in range(H_kv)], dtype=torch.int32,
                              device=dev)
    zone_c = (kn.contiguous(), vn.contiguous()) if counts is None else (kn, vn, counts)
    out, _ = decode_attn_fused(cache, q_all, rope=rope, zone_c=zone_c)
    return out


@dataclass
class _LayerWeights:
    """What one decoder layer contributes to a decode step (fast_decode.py:343-387): references
    to the model's own tensors except the two concatenations."""
    input_ln_weight: torch.Tensor
    input_ln_eps: float
    q_proj_weight: torch.Tensor
    k_proj_weight: torch.Tensor
    v_proj_weight: torch.Tensor
    o_proj_weight: torch.Tensor
    qkv_weight: torch.Tensor                  # [q_dim + 2 * kv_dim, hidden]: one GEMV for q, k, v
    qkv_split_sizes: Tuple[int, int, int]
    qkv_bias: Optional[torch.Tensor]          # None when the projections have no bias (Llama, Qwen3)
    post_ln_weight: torch.Tensor
    post_ln_eps: float
    gate_up_weight: torch.Tensor              # [2 * intermediate, hidden]
    gate_up_split_sizes: Tuple[int, int]
    down_proj_weight: torch.Tensor
    q_norm_weight: Optional[torch.Tensor] = None   # per-head q / k RMSNorm (Qwen3), applied before RoPE
    k_norm_weight: Optional[torch.Tensor] = None
    qk_norm_eps: float = 1e-5
    device: Optional[torch.device] = None


@dataclass
class PreExtractedWeights:
    """fast_decode.py:389-415 for a model that lives on one GPU."""
    embed_tokens: object
    final_norm_weight: torch.Tensor
    final_norm_eps: float
    lm_head_weight: torch.Tensor
    rotary_emb: object
    layers: List[_LayerWeights] = field(default_factory=list)
    num_layers: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    hidden_size: int = 0
    attn_output_dim: int = 0
    num_kv_groups: int = 0
    device: Optional[torch.device] = None


def pre_extract_weights(model) -> PreExtractedWeights:
    """Collect the weights of a Llama-style ``*ForCausalLM`` once (fast_decode.py:418-621): layer
    norms, q/k/v projections concatenated into one matrix (biases too where the model has them),
    gate and up projections concatenated, optional per-head q/k norms, embedding, final norm, LM
    head and the rotary module.  The result is cached on the model.  All parameters must be on
    one device: this build drives a single GPU."""
    cached = getattr(model, "_obkv_pre_extracted_weights", None)
    if cached is not None:
        return cached
    cfg = model.config
    devices = {p.device for p in model.parameters() if p.device.type != "meta"}
    assert len(devices) == 1, f"the model must live on one device, found {sorted(map(str, devices))}"
    H_q, H_kv = cfg.num_attention_heads, cfg.num_key_value_heads
    head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // H_q
    layers: List[_LayerWeights] = []
    for layer in model.model.layers:
        attn, mlp = layer.self_attn, layer.mlp
        proj = (attn.q_proj, attn.k_proj, attn.v_proj)
        biases = [getattr(m, "bias", None) for m in proj]
        qkv_bias = None
        if any(b is not None for b in biases):
            qkv_bias = torch.cat([b if b is not None else m.weight.new_zeros(m.weight.shape[0])
                                  for b, m in zip(biases, proj)])
        q_norm, k_norm = getattr(attn, "q_norm", None), getattr(attn, "k_norm", None)
        layers.append(_LayerWeights(
            input_ln_weight=layer.input_layernorm.weight, input_ln_eps=layer.input_layernorm.variance_epsilon,
            q_proj_weight=attn.q_proj.weight, k_proj_weight=attn.k_proj.weight, v_proj_weight=attn.v_proj.weight,
            o_proj_weight=attn.o_proj.weight,
            qkv_weight=torch.cat([m.weight for m in proj]), qkv_split_sizes=tuple(m.weight.shape[0] for m in proj),
            qkv_bias=qkv_bias,
            post_ln_weight=layer.post_attention_layernorm.weight,
            post_ln_eps=layer.post_attention_layernorm.variance_epsilon,
            gate_up_weight=torch.cat([mlp.gate_proj.weight, mlp.up_proj.weight]),
            gate_up_split_sizes=(mlp.gate_proj.weight.shape[0], mlp.up_proj.weight.shape[0]),
            down_proj_weight=mlp.down_proj.weight,
            q_norm_weight=None if q_norm is None else q_norm.weight,
            k_norm_weight=None if k_norm is None else k_norm.weight,
            qk_norm_eps=getattr(q_norm, "variance_epsilon", 1e-5) if q_norm is not None else 1e-5,
            device=attn.q_proj.weight.device))
    rotary = getattr(model.model, "rotary_emb", None)
    if rotary is None:
        rotary = model.model.layers[0].self_attn.rotary_emb
    weights = PreExtractedWeights(
        embed_tokens=model.model.embed_tokens, final_norm_weight=model.model.norm.weight,
        final_norm_eps=model.model.norm.variance_epsilon, lm_head_weight=model.lm_head.weight, rotary_emb=rotary,
        layers=layers, num_layers=len(layers), num_heads=H_q, num_kv_heads=H_kv, head_dim=head_dim,
        hidden_size=cfg.hidden_size, attn_output_dim=H_q * head_dim, num_kv_groups=H_q // H_kv,
        device=next(iter(devices)))
    model._obkv_pre_extracted_weights = weights
    return weights


class _DecodeStep:
    """One greedy decode step over device-resident state, written so that the same calls run
    eagerly or are captured once into a HIP graph: the token, its position, the zone C write row
    and the zone C token counts live in device tensors that the step itself advances, so a replay
    needs no argument from the host.  Per layer, six launches: q/k/v GEMV with the residual add
    and RMSNorm folded into the staging of its input row, zones A+B+C attention (two launches: q
    rotated while the streaming kernel stages it; the merge launch rotates k and appends the fp32
    K|V row to zone C first), output projection (its fp32 input rounded to the model type while it is staged), gate/up
    GEMV (residual add + RMSNorm folded in), down projection (SiLU * up folded in)."""

    def __init__(self, W: PreExtractedWeights, caches: List[StreamCache], new_kv_buf: List[torch.Tensor],
                 dtype: torch.dtype):
        dev = W.device
        self.W, self.caches, self.new_kv_buf, self.dtype = W, caches, new_kv_buf, dtype
        self.token = torch.zeros(1, 1, dtype=torch.long, device=dev)
        self.position = torch.zeros(1, 1, dtype=torch.long, device=dev)
        self.write_row = torch.zeros(1, dtype=torch.long, device=dev)
        self.n_new = torch.zeros(W.num_kv_heads, dtype=torch.int32, device=dev)   # tokens in zone C, this one included
        self.attn_out = torch.empty(W.num_heads, W.head_dim, dtype=torch.float32, device=dev)
        self.lse = torch.empty(W.num_heads, dtype=torch.float32, device=dev)
        self.hidden = None      # final-normalized hidden state [1,1,hidden] of the last step
        self.logits = None      # [1,1,vocab] of the last step

    def reset(self, token: torch.Tensor, position: int) -> None:
        self.token.copy_(token.reshape(1, 1))
        self.position.fill_(position)
        self.write_row.zero_()
        self.n_new.fill_(1)

    def run(self) -> None:
        W = self.W
        D = W.head_dim
        h = W.embed_tokens(self.token)                                   # [1,1,hidden], the residual stream
        cos, sin = W.rotary_emb(h, self.position)
        rope = (cos.view(D)[:D // 2], sin.view(D)[:D // 2])
        delta = None                                                     # branch output not yet added to h
        for lw, cache, buf in zip(W.layers, self.caches, self.new_kv_buf):
            qkv, h = _norm_linear_row(h, delta, lw.input_ln_weight, lw.input_ln_eps, lw.qkv_weight, lw.qkv_bias)
            q, k, v = qkv.split(lw.qkv_split_sizes, dim=-1)
            q_2d, k_2d, v_2d = q.view(W.num_heads, D), k.view(W.num_kv_heads, D), v.view(W.num_kv_heads, D)
            if lw.q_norm_weight is not None:
                q_2d = _rms_norm(q_2d, lw.q_norm_weight, lw.qk_norm_eps)
            if lw.k_norm_weight is not None:
                k_2d = _rms_norm(k_2d, lw.k_norm_weight, lw.qk_norm_eps)
            rows = buf[0]                                                # [H_kv, capacity, 2D] fp32, K | V
            decode_attn_fused(cache, q_2d, out=self.attn_out, lse=self.lse, rope=rope,   # q rotated while staged
                              zone_c=(rows[:, :, :D], rows[:, :, D:], self.n_new),
                              append=(k_2d, v_2d, self.write_row))        # k rotated + appended by the merge launch
            o = _linear_row(self.attn_out.view(1, 1, W.attn_output_dim), lw.o_proj_weight)     # fp32 in, rounded inside
            gate_up, h = _norm_linear_row(h, o, lw.post_ln_weight, lw.post_ln_eps, lw.gate_up_weight)
            gate, up = gate_up.split(lw.gate_up_split_sizes, dim=-1)
            delta = _silu_linear_row(gate, up, lw.down_proj_weight)
        self.hidden = _rms_norm(h, W.final_norm_weight, W.final_norm_eps, delta=delta, residual_out=h)
        self.logits = _linear_row(self.hidden, W.lm_head_weight)
        _argmax_advance(self.logits, self.token, self.position, self.write_row, self.n_new)


def _layer_stream_caches(dual_cache, num_kv_groups: int) -> List[StreamCache]:
    """One streaming cache per layer (a sequential model attends layer by layer), built once per
    packed cache and kept on it like the reference keeps its pre-squeezed views."""
    caches = getattr(dual_cache, "_stream_caches", None)
    if caches is None or len(caches) != len(dual_cache.packed):
        v16 = list(dual_cache.new_v_only) if dual_cache.new_v_only is not None else [None] * len(dual_cache.packed)
        caches = [build_stream_cache([(pl, nvo)], num_kv_groups) for pl, nvo in zip(dual_cache.packed, v16)]
        dual_cache._stream_caches = caches
    return caches


def greedy_decode_fast(model, dual_cache, next_token_logits, max_new_tokens, eos_token_ids, primary_device,
                       decode_position_start, use_cuda_graph=False, return_logits=False,
                       next_token_hidden=None, logits_observer=None, hidden_observer=None):
    """Greedy decode over a packed prompt cache without ``model.forward`` (fast_decode.py:731-1860):
    same arguments, return value, observer protocol and errors.

    The first token is the argmax of ``next_token_logits``; every step then consumes the pending
    token (observers see ``(step, logits | hidden, token, is_eos)`` first; an EOS token ends the
    loop without being returned), runs the model for it at position ``decode_position_start +
    step`` and takes the argmax of the new logits.  Attention reads the packed prompt through the
    streaming layout (built on first use, cached on ``dual_cache``) and the tokens generated so
    far from fp32 zone C buffers (cached on ``dual_cache`` under the reference's attribute name).

    ``use_cuda_graph``: step 0 runs eagerly, then the whole step - every layer, LM head and argmax
    - is captured as ONE HIP graph and replayed; token, position and zone C length are device
    state that the graph advances, so no per-length or per-layer graphs are needed.  As in the
    reference, observers and ``return_logits`` need the eager path."""
    eos_set = {int(t) for t in eos_token_ids if t is not None}
    if (return_logits or logits_observer is not None or hidden_observer is not None) and use_cuda_graph:
        raise NotImplementedError("logit observation is only supported under eager decode (use_cuda_graph=False)")
    if hidden_observer is not None and next_token_hidden is None:
        raise ValueError("hidden_observer requires next_token_hidden")
    W = pre_extract_weights(model)
    dev = torch.device(primary_device)
    _lib.require_device(W.lm_head_weight)
    assert W.head_dim == 128, f"the packed format is defined for head_dim 128, got {W.head_dim}"
    assert len(dual_cache.packed) == W.num_layers, "one packed layer per decoder layer"
    model_dtype = next(model.parameters()).dtype
    caches = _layer_stream_caches(dual_cache, W.num_kv_groups)

    key = (max_new_tokens, W.num_kv_heads, W.head_dim, str(dev), W.num_layers)
    kept = getattr(dual_cache, "_new_kv_buf_cache", None)
    if kept is not None and kept.get("key") == key:
        new_kv_buf = kept["buffers"]
    else:
        new_kv_buf = [torch.zeros(1, W.num_kv_heads, max(max_new_tokens, 1), 2 * W.head_dim, dtype=torch.float32,
                                  device=dev) for _ in range(W.num_layers)]
        dual_cache._new_kv_buf_cache = {"key": key, "buffers": new_kv_buf}

    if next_token_logits.dim() == 1:
        next_token_logits = next_token_logits.unsqueeze(0)
    generated: List[int] = []
    collected = [] if return_logits else None
    step_state = _DecodeStep(W, caches, new_kv_buf, model_dtype)
    graph = None
    with torch.inference_mode():
        step_state.reset(next_token_logits.argmax(dim=-1, keepdim=True).to(dev), int(decode_position_start))
        for step in range(max_new_tokens):
            token_id = int(step_state.token.item())
            if logits_observer is not None:
                logits_observer(step, next_token_logits if step == 0 else step_state.logits[:, -1, :], token_id,
                                token_id in eos_set)
            if hidden_observer is not None:
                hidden_observer(step, next_token_hidden if step == 0 else step_state.hidden[:, -1, :], token_id,
                                token_id in eos_set)
            if token_id in eos_set:
                break
            generated.append(token_id)
            if use_cuda_graph and step >= 1:
                if graph is None:       # step 0 warmed every library and workspace; record the step once
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        step_state.run()
                graph.replay()
            else:
                step_state.run()
            if collected is not None:
                collected.append(step_state.logits[:, -1, :].detach().float().clone().cpu())
    if return_logits:
        return generated, collected
    return generated
