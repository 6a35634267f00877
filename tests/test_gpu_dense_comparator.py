"""The dense fp16 decode-attention kernel the benchmark prices the packed path against
(``rdkv_probe_dense_decode``): a floating-point kernel, checked against the plain fp32 tensor
expression of the same attention."""
import pytest
import torch

from rdkv_amd import _lib
from tests.gpu_util import DEV, require_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    require_gpu()


@pytest.mark.parametrize("T,H_kv,G,chunks", [(4096, 8, 4, 64), (1000, 2, 4, 7), (33, 1, 8, 64), (5000, 3, 8, 16),
                                             (1, 2, 4, 4), (32768, 8, 4, 64)])
def test_dense_decode_matches_fp32_attention(T, H_kv, G, chunks):
    """softmax(q.K^T / sqrt(128)).V per query head against fp32 tensor expressions over the same fp16
    inputs; tolerance 2e-3 absolute and 1e-2 of the largest reference value (the attention
    tolerance of the packed path; the kernel's own error is the fp16 dot products' 1e-3)."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(T + G)
    K = torch.randn(H_kv, T, 128, generator=g).half().to(DEV)
    V = torch.randn(H_kv, T, 128, generator=g).half().to(DEV)
    q = torch.randn(H_kv * G, 128, generator=g).half().to(DEV)
    out = torch.empty(H_kv * G, 128, dtype=torch.float32, device=DEV)
    ws = torch.empty(lib.rdkv_probe_dense_decode_workspace_bytes(H_kv * G, chunks), dtype=torch.uint8, device=DEV)
    _lib.check(lib.rdkv_probe_dense_decode(q.data_ptr(), K.data_ptr(), V.data_ptr(), T, H_kv, G, chunks,
                                           out.data_ptr(), ws.data_ptr(), ws.numel(),
                                           _lib.stream_of(torch.device(DEV))))
    s = torch.einsum("hgd,htd->hgt", q.float().view(H_kv, G, 128), K.float()) / 128 ** 0.5
    ref = torch.einsum("hgt,htd->hgd", torch.softmax(s, dim=-1), V.float()).reshape(H_kv * G, 128)
    err = float((out - ref).abs().max())
    assert torch.isfinite(out).all()
    assert err <= 2e-3 and err <= 1e-2 * float(ref.abs().max()), f"max-abs error {err:.3e}"


def test_dense_decode_rejects_what_it_cannot_take():
    lib = _lib.load()
    x = torch.zeros(8, 128, dtype=torch.float16, device=DEV)
    out = torch.empty(8, 128, dtype=torch.float32, device=DEV)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    st = _lib.stream_of(torch.device(DEV))
    assert lib.rdkv_probe_dense_decode(x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 2, 3, 4, out.data_ptr(),
                                       ws.data_ptr(), ws.numel(), st) == _lib.RDKV_EINVAL      # G = 3
    assert lib.rdkv_probe_dense_decode(x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, 2, 4, 4, out.data_ptr(),
                                       ws.data_ptr(), 16, st) == _lib.RDKV_EWORKSPACE
