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


class _OracleEngine:
    """The CPU oracle behind the engine interface the decoder harness uses (prefill / decode / len,
    ``last_attn``): the checker in the place of the HIP engine, same module, same inputs."""

    def __init__(self, oracle, init, **kw):
        self.orc = oracle.OracleLayer(num_lite_tokens=kw["num_lite_tokens"], attn_topk=kw["attn_topk"],
                                      num_key_value_groups=kw["num_key_value_groups"], r=kw["r"], max_iter=kw["max_iter"],
                                      tol=kw["tol"], capacity=kw["capacity"], compute_dtype=torch.float64)
        self.oracle, self.init = oracle, init
        self.attn_in_step, self.last_attn = True, None
        self.selected = []

    def prefill(self, query_states, key_states, value_states):
        self.orc.prefill(query_states.cpu(), key_states.cpu(), value_states.cpu(), A_Q0=self.init[0], A_K0=self.init[1])

    def decode(self, q, k, v):
        K, V = self.orc.decode(q.cpu(), k.cpu(), v.cpu())
        self.last_attn = self.oracle.attention(q.cpu(), K, V, torch.float64).to(q.dtype).to(q.device)
        if self.orc.hit_indices is not None:
            self.selected.append(self.orc.hit_indices[..., 0].clone())
        return K.to(q.device), V.to(q.device)

    def __len__(self):
        return len(self.orc)


def test_selection_path_against_oracle_run(dec, oracle):
    """The same module decoded twice -- with the HIP engines and with the CPU oracle in their place (same injected
    initial factors) -- over a prompt that goes through the selection path (l > k + lite): the greedy tokens must be
    identical, and every layer's resident sets must agree step by step (the two runs evolve independently, so a
    score within rounding of the threshold may swap one token: at least 15 of 16 per head, and the sets of the last
    step are printed)."""
    print("decoder: selection path vs oracle-driven run", flush=True)
    import lrqk_amd
    m = _model(dec)
    g = torch.Generator().manual_seed(1)
    b, l, new = 2, 64, 12
    ids = torch.randint(0, 97, (b, l), generator=g).to(DEV)
    kw = dict(r=4, num_active_tokens=16, lite_tokens=4, max_iter=(2, 2), tol=(1e-8, 1e-8), max_sequence_length=32)
    inits = [(torch.randn((b, 4, l, 4), generator=g), torch.randn((b, 4, l, 4), generator=g)) for _ in range(2)]


    class Recording(lrqk_amd.LightAttentionIndicesFactory):
        def decode(self, q, k, v):
            out = super().decode(q, k, v)
            if self.hit_indices is not None:
                self.selected.append(self.hit_indices[..., 0].cpu().clone())
            return out

    made = []

    def hip_factory(**a):
        e = Recording(**a)
        e.init_factors = inits[len(made)]
        e.selected = []
        made.append(e)
        return e

    cache = m.new_cache(**kw)
    cache.lwattn.default_factory = lambda: hip_factory(num_lite_tokens=4, attn_topk=16, num_key_value_groups=2, r=4,
                                                       max_iter=(2, 2), tol=(1e-8, 1e-8), capacity=32)
    got, *_ = m.generate(ids, new, cache)

    omade = []

    def orc_factory():
        e = _OracleEngine(oracle, inits[len(omade)], num_lite_tokens=4, attn_topk=16, num_key_value_groups=2, r=4,
                          max_iter=(2, 2), tol=(1e-8, 1e-8), capacity=32)
        omade.append(e)
        return e

    ocache = m.new_cache(**kw)
    ocache.lwattn.default_factory = orc_factory
    want, *_ = m.generate(ids, new, ocache)
    assert torch.equal(got.cpu(), want.cpu()), (got.cpu().tolist(), want.cpu().tolist())
    worst = 16
    for li in range(2):
        assert len(made[li].selected) == len(omade[li].selected) == new - 1
        for step, (a, o) in enumerate(zip(made[li].selected, omade[li].selected)):
            for ra, ro in zip(a.reshape(-1, 16).tolist(), o.reshape(-1, 16).tolist()):
                common = len(set(ra) & set(ro))
                worst = min(worst, common)
                assert common >= 15, (li, step, sorted(ra), sorted(ro))
    print("   tokens identical; smallest agreement of a head's resident set with the oracle run: %d of 16" % worst,
          flush=True)
