"""The attention entry point that allocates nothing (lrqk_attention_static) against the
ordinary one (lrqk_attention): same kernels, so the outputs must be bit-identical.  Two calls in
a row share the library's fixed block of partial results; the second is smaller, so it finds
the first call's leftovers there."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(ops, ws, seed, b, H, n, d, n_valid, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((b, H, 1, d), generator=g).to(dtype).to(DEV)
    K = torch.randn((b, H, n, d), generator=g).to(dtype).to(DEV)
    V = torch.randn((b, H, n, d), generator=g).to(dtype).to(DEV)
    exp = ops.attention(ws, q, K, V, n_valid)
    out = torch.full((b, H, 1, d), float("nan"), dtype=dtype, device=DEV)
    # one call first: the library resolves the address of its fixed block on a device's first call (and the
    # runtime loads the kernels); the calls measured below must then leave the device's free memory untouched --
    # hipMemGetInfo sees a hipMalloc inside the library, which torch's own allocator counters would not
    ops.attention_static(q, K, V, out, n_valid)
    torch.cuda.synchronize()
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    ops.attention_static(q, K, V, out, n_valid)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the entry point changed the device's free memory"
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, exp), (seed, float((out.float() - exp.float()).abs().max()))
    return q, K, V, out


def test_static_attention_matches_and_reuses_its_block(oracle):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lrqk_amd import ops, _lib
    ws = ops.Workspace()
    print("static attention: llama shape bf16, then a smaller fp32 call", flush=True)
    # first call: the decode shape (32 heads, 2112 slots, d 128, bf16): 32 x 33 splits
    _case(ops, ws, 0, 1, 32, 2112, 128, None, torch.bfloat16)
    # second call, smaller in every respect (fewer heads, fewer splits, some slots not valid)
    q, K, V, out = _case(ops, ws, 1, 1, 4, 300, 64, 270, torch.float32)
    exp = oracle.attention(q.cpu(), K.cpu()[:, :, :270], V.cpu()[:, :, :270])
    rel = float((out.cpu().double() - exp).norm() / exp.norm())
    assert rel < 1e-4, rel   # and the shared kernels still match the textbook softmax
    # a third, larger again (b = 4: 128 heads)
    _case(ops, ws, 2, 4, 32, 2112, 128, None, torch.bfloat16)
    # beyond the fixed block: refused with a clear error, nothing launched
    big_q = torch.zeros((1, 4096, 1, 128), dtype=torch.float32, device=DEV)
    big_kv = torch.zeros((1, 4096, 128, 128), dtype=torch.float32, device=DEV)
    with pytest.raises(_lib.LrqkError, match="static block"):
        ops.attention_static(big_q, big_kv, big_kv, torch.empty_like(big_q))
