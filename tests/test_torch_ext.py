"""The compiled PyTorch extension module `retrieval_attention_cpp` (csrc/torch_ext.cpp), the counterpart of the
reference's bind.cpp module (bind.cpp:246-757): names and error behaviour without a GPU; on a GPU its ops against the
ctypes binding of the same C entry point (bit-identical output) and against the oracle."""
import numpy as np
import pytest
import torch

import oracle
import topk_attn_amd
from topk_attn_amd import _lib as L


def _ext():
    return topk_attn_amd.load_torch_extension()


def test_module_surface():
    m = _ext()
    assert m.__name__ == "retrieval_attention_cpp"
    for v in L.RA_VARIANTS:
        for k in L.RA_TOPKS:
            op = getattr(m, "retrieval_attention%s_%d" % (v, k))
            assert "(TopK=%d)" % k in op.__doc__
    assert callable(m.retrieval_attention)


def test_rejects_host_tensors_and_wrong_types():
    m = _ext()
    q, kv = torch.zeros(1, 32, 128, dtype=torch.half), torch.zeros(8192, 32, 128, dtype=torch.half)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        m.retrieval_attention_128(q, kv, kv, torch.zeros_like(q))
    with pytest.raises(TypeError):
        m.retrieval_attention_128(q, kv, kv)                      # output missing, as in the reference's signature


@pytest.mark.gpu
@pytest.mark.parametrize("variant,topk", [("", 128), ("_pipelined_global", 32), ("_gather_baseline", 1024)])
def test_ops_match_ctypes_binding_and_oracle(variant, topk):
    from tests.util import announce, bits_of
    from topk_attn_amd import retrieval_attention_cpp as ct
    announce("torch extension retrieval_attention%s_%d" % (variant, topk))
    m = _ext()
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    B = 3
    q = (torch.randn((B, 32, 128), generator=g, device="cuda") * 0.1).half()
    k = (torch.randn((8192, 32, 128), generator=g, device="cuda") * 0.1).half()
    v = (torch.randn((8192, 32, 128), generator=g, device="cuda") * 0.1).half()
    out_ext, out_ct = torch.zeros_like(q), torch.zeros_like(q)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                 # the op follows PyTorch's current stream
        getattr(m, "retrieval_attention%s_%d" % (variant, topk))(q, k, v, out_ext)
    side.synchronize()
    getattr(ct, "retrieval_attention%s_%d" % (variant, topk))(q, k, v, out_ct)
    torch.cuda.synchronize()
    assert torch.equal(out_ext.view(torch.int16), out_ct.view(torch.int16))
    qb, kb, vb = bits_of(q), bits_of(k), bits_of(v)
    for h in (0, 31):
        ref, _, _ = oracle.retrieval_attention(qb[1, h], kb[:, h], vb[:, h], oracle.F16, 4, topk, 1.0)
        assert np.abs(out_ext[1, h].float().cpu().numpy() - ref).max() < 2e-3
    with pytest.raises(RuntimeError, match="expected scalar type Half"):
        m.retrieval_attention_128(q.float(), k.float(), v.float(), out_ext.float())
    with pytest.raises(RuntimeError, match="8192"):
        m.retrieval_attention_128(q, k[:4096], v[:4096], out_ext)


@pytest.mark.gpu
def test_generic_op_bf16():
    from tests.util import announce
    from topk_attn_amd import ops
    announce("torch extension generic op bf16, 2 chunks of 1000 keys, top 50")
    m = _ext()
    g = torch.Generator(device="cuda")
    g.manual_seed(8)
    q = (torch.randn((2, 4, 128), generator=g, device="cuda") * 0.1).bfloat16()
    k = (torch.randn((2000, 4, 128), generator=g, device="cuda") * 0.1).bfloat16()
    v = (torch.randn((2000, 4, 128), generator=g, device="cuda") * 0.1).bfloat16()
    a, b = torch.zeros_like(q), torch.zeros_like(q)
    m.retrieval_attention(q, k, v, a, 50, num_chunks=2, scale=0.5)
    ops.retrieval_attention(q, k, v, b, 50, 2, 0.5)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
