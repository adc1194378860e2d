"""GPT-2-shaped greedy decode through the C ABI against the oracle's composition of the same ops (BASELINE config 5 at
sizes the oracle finishes in seconds)."""
import numpy as np
import pytest

from deeplearning4j_amd.decoder import Decoder, DecoderConfig, init_weights
from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32

pytestmark = pytest.mark.gpu

SMALL = dict(n_layer=2, d_model=128, n_head=2, d_ff=256, vocab=1000, max_len=64)


@pytest.mark.parametrize("batch,prompt", [(1, 16), (3, 16), (2, 1)])
def test_decode_fp32_ids_bit_exact(ex, oracle, batch, prompt):
    from oracle.decoder_oracle import OracleDecoder
    cfg = DecoderConfig(**SMALL)
    w = init_weights(cfg, 5005)
    ids = np.random.default_rng(5005 + batch).integers(0, cfg.vocab, (batch, prompt))
    want = OracleDecoder(cfg, w, oracle.FLOAT32, batch=batch)
    want_ids = want.generate(ids, 8)
    dec = Decoder(cfg, w, FLOAT32, batch=batch, executioner=ex)
    got_ids = dec.generate(ids, 8)
    assert got_ids.dtype == np.int64
    assert (got_ids == want_ids).all()
    # fp32 mmul/attention gate: 1e-4
    np.testing.assert_allclose(dec.logits(1), want.last_logits, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("batch", [1, 4])
def test_decode_bf16_logits_and_ids(ex, oracle, batch):
    from oracle.decoder_oracle import OracleDecoder
    cfg = DecoderConfig(**SMALL)
    w = init_weights(cfg, 5005)
    ids = np.random.default_rng(77 + batch).integers(0, cfg.vocab, (batch, 24))
    want = OracleDecoder(cfg, w, oracle.BFLOAT16, batch=batch)
    dec = Decoder(cfg, w, BFLOAT16, batch=batch, executioner=ex)
    # teacher-forced: both sides consume the oracle's tokens, logits are compared at every step (bf16 gate 1e-2)
    nxt = want.forward(ids)
    got = dec.forward(ids)
    for step in range(6):
        lg_w, lg_g = want.last_logits, dec.logits()
        np.testing.assert_allclose(lg_g, lg_w, rtol=1e-2, atol=1e-2)
        # ids agree wherever the oracle's top-2 gap is wider than the bf16 resolution of the logits
        top2 = np.sort(lg_w, axis=1)[:, -2:]
        decided = (top2[:, 1] - top2[:, 0]) > 2e-2 * np.maximum(1.0, np.abs(top2[:, 1]))
        g = got.to_numpy()
        assert (g[decided] == nxt[decided]).all()
        feed = nxt.reshape(batch, 1)
        nxt = want.forward(feed)
        got = dec.forward(feed)


def test_decode_head_dim_64_uses_fused_attention(ex):
    """bf16, d_head 64: prefill and decode steps run end to end and are deterministic across two runs."""
    cfg = DecoderConfig(**SMALL)
    w = init_weights(cfg, 9)
    ids = np.random.default_rng(9).integers(0, cfg.vocab, (2, 20))
    dec = Decoder(cfg, w, BFLOAT16, batch=2, executioner=ex)
    a = dec.generate(ids, 5)
    b = dec.generate(ids, 5)
    assert (a == b).all()


@pytest.mark.parametrize("replay_mode", [0, 1])
def test_graph_replay_matches_eager_steps(ex, replay_mode):
    """Decode steps recorded as HIP graphs: the first generation records one graph per cache length, the second replays
    them; eager op-by-op work and synchronisations sit between the replays, and every generation must reproduce the
    eager ids bit for bit (a replayed kernel runs with exactly the recorded arguments).  Both ways of replaying: the
    instantiated graph (0) and the merged sequence launched kernel by kernel by the library (1)."""
    from deeplearning4j_amd.decoder import Decoder, DecoderConfig, init_weights
    from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, HALF
    ex.L.nd4jhipSetGraphReplayMode(replay_mode)
    assert ex.L.nd4jhipGetGraphReplayMode() == replay_mode
    try:
        _graph_replay_matches_eager_steps(ex, Decoder, DecoderConfig, init_weights, BFLOAT16, HALF, FLOAT32)
    finally:
        ex.L.nd4jhipSetGraphReplayMode(0)


def _graph_replay_matches_eager_steps(ex, Decoder, DecoderConfig, init_weights, BFLOAT16, HALF, FLOAT32):
    cfg = DecoderConfig(vocab=512, d_model=128, n_head=2, n_layer=2, max_len=96)
    w = init_weights(cfg, seed=5)
    rng = np.random.default_rng(6)
    for dtype in (HALF, BFLOAT16, FLOAT32):    # fp32: the streaming attention kernel takes the single-token steps, nothing allocates
        for batch in (1, 3):
            prompt = rng.integers(0, cfg.vocab, (batch, 17))
            eager = Decoder(cfg, w, dtype, batch=batch, executioner=ex)
            want = eager.generate(prompt, 24)
            dec = Decoder(cfg, w, dtype, batch=batch, executioner=ex)
            dec.use_graphs = True
            first = dec.generate(prompt, 24)                   # records
            assert np.array_equal(first, want)
            assert len(dec._graphs) == 23
            other = eager.generate(rng.integers(0, cfg.vocab, (batch, 17)), 5)      # unrelated eager work in between
            again = dec.generate(prompt, 24)                   # replays every graph
            assert np.array_equal(again, want)
            assert len(dec._graphs) == 23
            prompt2 = rng.integers(0, cfg.vocab, (batch, 17))  # same lengths, other tokens: replay on new data
            assert np.array_equal(dec.generate(prompt2, 24), eager.generate(prompt2, 24))
            dec.close()
            assert other.shape == (batch, 5)
