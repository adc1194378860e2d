"""BASELINE config 5 at its real shape: GPT-2-small (12 layers, d_model 768, 12 heads, d_ff 3072, vocab 50257) through the
C ABI against the oracle's composition of the same ops.

  * fp32: greedy ids bit for bit and logits at the fp32 mmul / attention gate (1e-4), for a 32-token prompt + 8 steps and
    for the 512-token prefill;
  * bf16: teacher-forced logits, batch 1 and 32, gated by the oracle's own bf16-against-fp32 deviation at this depth;
  * decode steps replayed as HIP graphs reproduce the eager ids and logits, also on new tokens (batch 1, 8 and 32).
The oracle runs on the host cores, so prompts stay short where the batch is large.
"""
import numpy as np
import pytest

from deeplearning4j_amd.decoder import Decoder, DecoderConfig, init_weights
from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpt2():
    cfg = DecoderConfig(max_len=576)          # GPT-2-small everywhere else; a shorter position table keeps the caches small
    assert (cfg.n_layer, cfg.d_model, cfg.n_head, cfg.d_ff, cfg.vocab) == (12, 768, 12, 3072, 50257)
    return cfg, init_weights(cfg, 5005)


def test_gpt2_small_fp32_ids_bit_exact(ex, oracle, gpt2):
    from oracle.decoder_oracle import OracleDecoder
    cfg, w = gpt2
    ids = np.random.default_rng(5005).integers(0, cfg.vocab, (1, 32))
    want = OracleDecoder(cfg, w, oracle.FLOAT32, batch=1)
    want_ids = want.generate(ids, 8)
    dec = Decoder(cfg, w, FLOAT32, batch=1, executioner=ex)
    got_ids = dec.generate(ids, 8)
    assert np.array_equal(got_ids, want_ids)
    np.testing.assert_allclose(dec.logits(1), want.last_logits, rtol=1e-4, atol=1e-4)


def test_gpt2_small_fp32_prefill_512(ex, oracle, gpt2):
    from oracle.decoder_oracle import OracleDecoder
    cfg, w = gpt2
    ids = np.random.default_rng(512).integers(0, cfg.vocab, (1, 512))
    want = OracleDecoder(cfg, w, oracle.FLOAT32, batch=1)
    want_next = want.forward(ids)
    dec = Decoder(cfg, w, FLOAT32, batch=1, executioner=ex)
    got_next = dec.forward(ids).to_numpy()
    assert np.array_equal(got_next, want_next)
    np.testing.assert_allclose(dec.logits(512), want.last_logits, rtol=1e-4, atol=1e-4)
    # and two cached steps on top of the 512-token history (50257-wide argmax, attention over the cache)
    for _ in range(2):
        want_next = want.forward(want_next.reshape(1, 1))
        got_next = dec.forward(None).to_numpy()
        assert np.array_equal(got_next, want_next)
    np.testing.assert_allclose(dec.logits(1), want.last_logits, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("batch,prompt,steps", [(1, 64, 4), (32, 6, 3)])
def test_gpt2_small_bf16_teacher_forced_logits(ex, oracle, gpt2, batch, prompt, steps):
    """bf16 at depth 12.  The 1e-2 gate is a per-op gate (the 2-layer model of test_decoder_gpu.py is held to it); through
    12 layers x 13 rounded ops two correct bf16 evaluations that sum in different orders drift apart by more than that.
    The yardstick here is the oracle itself: `noise` = how far its own bf16 run lands from its fp32 run on the same
    tokens.  The device's bf16 logits must be as close to the fp32 logits as the oracle's bf16 logits are (x 1.5), and
    within twice that of the oracle's bf16 logits."""
    from oracle.decoder_oracle import OracleDecoder
    cfg, w = gpt2
    ids = np.random.default_rng(77 + batch).integers(0, cfg.vocab, (batch, prompt))
    want = OracleDecoder(cfg, w, oracle.BFLOAT16, batch=batch)
    ref32 = OracleDecoder(cfg, w, oracle.FLOAT32, batch=batch)
    dec = Decoder(cfg, w, BFLOAT16, batch=batch, executioner=ex)
    nxt = want.forward(ids)
    ref32.forward(ids)
    got = dec.forward(ids)
    for step in range(steps):
        lg_w, lg_32, lg_g = want.last_logits, ref32.last_logits, dec.logits()
        noise = float(np.abs(lg_w - lg_32).max())
        assert 1e-3 < noise < 0.1, noise
        assert float(np.abs(lg_g - lg_32).max()) <= 1.5 * noise, (step, noise)
        assert float(np.abs(lg_g - lg_w).max()) <= 2.0 * noise, (step, noise)
        # ids agree wherever the fp32 top-2 gap is wider than that noise
        top2 = np.sort(lg_32, axis=1)[:, -2:]
        decided = (top2[:, 1] - top2[:, 0]) > 4.0 * noise
        g = got.to_numpy()
        assert (g[decided] == lg_32.argmax(1)[decided]).all()
        feed = nxt.reshape(batch, 1)
        nxt = want.forward(feed)
        ref32.forward(feed)
        got = dec.forward(feed)


@pytest.mark.parametrize("batch,replay_mode", [(1, 0), (8, 0), (32, 0), (1, 1), (32, 1)])
def test_gpt2_small_graph_replay_matches_eager(ex, gpt2, batch, replay_mode):
    """Recorded steps against eager steps at the real shape: ids and the logits read back after a replay (the replay must
    stamp the buffers it writes, or the host would keep serving the previous copy); replayed as graphs (0) and as the
    merged sequence launched kernel by kernel (1)."""
    ex.L.nd4jhipSetGraphReplayMode(replay_mode)
    try:
        _gpt2_small_graph_replay_matches_eager(ex, gpt2, batch)
    finally:
        ex.L.nd4jhipSetGraphReplayMode(0)


def _gpt2_small_graph_replay_matches_eager(ex, gpt2, batch):
    cfg, w = gpt2
    rng = np.random.default_rng(batch)
    prompt = rng.integers(0, cfg.vocab, (batch, 24))
    eager = Decoder(cfg, w, BFLOAT16, batch=batch, executioner=ex)
    want = eager.generate(prompt, 6)
    want_logits = eager.logits(1)
    dec = Decoder(cfg, w, BFLOAT16, batch=batch, executioner=ex)
    dec.use_graphs = True
    assert np.array_equal(dec.generate(prompt, 6), want)                     # records
    assert np.array_equal(dec.logits(1), want_logits)
    # the recorded steps went through the merging pass: per layer the two residual Adds, the GELU after the first feed-forward
    # product and the two cache writes after the qkv product ride in a product's epilogue, and the two layer norms are
    # computed by the products that consume them
    fused = [ex.L.nd4jhipGraphFusedOps(g) for g in dec._graphs.values()]
    assert fused and min(fused) == 7 * cfg.n_layer, fused
    # ... and every one of them did run inside its neighbour's kernel (no merged step fell back to separate launches)
    assert [ex.L.nd4jhipGraphFusedApplied(g) for g in dec._graphs.values()] == fused
    # every kernel node of every recorded step within the limits the runtime reports for its function (host-side walk)
    for g in dec._graphs.values():
        assert ex.L.nd4jhipGraphAudit(g) == 0, ex.L.lastErrorMessage()
    stale = dec.logits(1)                                                   # host copy read: a later replay must refresh it
    prompt2 = rng.integers(0, cfg.vocab, (batch, 24))
    want2 = eager.generate(prompt2, 6)
    want2_logits = eager.logits(1)
    assert np.array_equal(dec.generate(prompt2, 6), want2)                   # replays on new tokens
    got2_logits = dec.logits(1)
    assert np.array_equal(got2_logits, want2_logits)
    assert not np.array_equal(got2_logits, stale)
    dec.close()
