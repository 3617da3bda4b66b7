"""The decoder stack around the cache: with k + lite >= the whole sequence the LRQK run keeps every
token (growing-prefix branch) and must decode the same tokens as the dense-cache run of the same
module; with a short active set it must run the selection path end to end."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dec():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lrqk_amd import decoder
    return decoder


def _model(dec, dtype=torch.float32):
    cfg = dec.DecoderConfig(layers=2, hidden=64, heads=4, kv_heads=2, head_dim=16, intermediate=128, vocab=97,
                            rope_theta=1e4)
    return dec.LlamaShapeDecoder(cfg, dtype, DEV, seed=3)


def test_prefix_branch_equals_dense_cache(dec):
    print("decoder: prefix branch vs dense", flush=True)
    m = _model(dec)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, 97, (2, 24), generator=g).to(DEV)
    dense, *_ = m.generate(ids, 8, None)
    cache = m.new_cache(r=4, num_active_tokens=20, lite_tokens=12, max_iter=(2, 2), tol=(1e-8, 1e-8),
                        max_sequence_length=16)
    got, *_ = m.generate(ids, 8, cache)
    assert torch.equal(got.cpu(), dense.cpu())
    assert cache.get_seq_length(0) == 24 + 7 and len(cache) == 2


def test_selection_path_runs_end_to_end(dec):
    print("decoder: selection path", flush=True)
    m = _model(dec)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 97, (2, 64), generator=g).to(DEV)
    cache = m.new_cache(r=4, num_active_tokens=16, lite_tokens=4, max_iter=(2, 2), tol=(1e-8, 1e-8),
                        max_sequence_length=32)
    got, t_pre, t_dec, steps = m.generate(ids, 12, cache)
    assert got.shape == (2, 12) and int(got.min()) >= 0 and int(got.max()) < 97
    for li in range(2):
        eng = cache.lwattn[li]
        assert len(eng) == 64 + 11 and eng.last_attn is not None
        idx = eng.hit_indices[..., 0]
        assert idx.shape == (2, 4, 16) and int(idx.max()) < len(eng)
        # every head's resident set is duplicate-free
        assert all(len(set(row.tolist())) == 16 for row in idx.reshape(-1, 16).cpu())
