"""End-to-end synthetic decoder (BASELINE config 5 shape family, reduced) against the CPU oracle.

Teacher forcing: the oracle is fed the tokens the GPU produced, and the logits of every step are
compared. aion's arithmetic re-quantizes the activations to int8 in front of every matmul, which
is discontinuous: a perturbation p of an activation flips a fraction p/step of the int8 codes
(step = amax/127), so any difference upstream (f32 summation order, exp2 vs the CPU's polynomial
exp with 4e-5 relative error) reappears downstream at about sqrt(p * step) of rms. The tolerance
is therefore stated against the CPU path's own sensitivity: a second oracle run whose only change
is the exact exp in attention (attn_exact) gives `self`. After a few re-quantizations every
perturbation saturates near the quantization step itself (the map e -> sqrt(e * step) has the fixed
point e = step), so `self` is a few percent of rms(logits) already for a 3-layer model. The GPU
must be statistically indistinguishable from such a variant: mean error <= 2 x mean self + 1e-3,
worst <= 3 x worst self. Greedy tokens must agree wherever the oracle's top-2 logit gap exceeds
twice the observed error.
"""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


class OraclePair:
    """aion's CPU path (polynomial exp) and the same path with the exact exp in attention."""

    def __init__(self, orc, cfg):
        mk = lambda exact: orc.Decoder(cfg.layers, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.ffn, cfg.vocab,
                                       cfg.max_seq, eps=cfg.eps, rope_base=cfg.rope_base, wdtype=cfg.wdtype, threads=8,
                                       attn_exact=exact)
        self.ref, self.alt = mk(False), mk(True)

    def set_weight(self, name, data):
        self.ref.set_weight(name, data)
        self.alt.set_weight(name, data)

    def forward(self, tokens, pos):
        return self.ref.forward(tokens, pos), self.alt.forward(tokens, pos)


def build(gpu, orc, cfg, seed):
    oracle = OraclePair(orc, cfg)
    dec = Decoder(gpu, cfg, SyntheticWeights(cfg, seed), on_weight=oracle.set_weight)
    return dec, oracle


def check_step(tag, gpu_logits, gpu_tok, ref, alt):
    orc_tok, orc_logits = ref
    rms = float(np.sqrt((orc_logits.astype(np.float64) ** 2).mean()))
    err = float(np.abs(gpu_logits - orc_logits).max())
    self_err = float(np.abs(alt[1] - orc_logits).max())
    top2 = np.sort(orc_logits)[-2:]
    gap = float(top2[1] - top2[0])
    say("  %s: gpu max|err|/rms = %.2e, cpu self-sensitivity = %.2e, top-2 gap/rms = %.2e, tokens %d / %d"
        % (tag, err / rms, self_err / rms, gap / rms, gpu_tok, orc_tok))
    if gap > 2 * err:
        assert gpu_tok == orc_tok, tag
    return err / rms, self_err / rms


SMALL = dict(layers=3, hidden=512, heads=8, kv_heads=1, head_dim=64, ffn=1024, vocab=2048, max_seq=48)
MID = dict(layers=2, hidden=2048, heads=8, kv_heads=1, head_dim=256, ffn=8192, vocab=8192, max_seq=64)


@pytest.mark.parametrize("shape,wdtype", [(SMALL, be.Q4_0), (SMALL, be.Q8_0), (MID, be.Q4_0)])
def test_prefill_then_greedy_decode_teacher_forced(gpu, orc, shape, wdtype):
    cfg = DecoderConfig(wdtype=wdtype, **shape)
    say("decoder", shape, wdtype)
    dec, oracle = build(gpu, orc, cfg, seed=5)
    try:
        rng = np.random.default_rng(9)
        prompt = rng.integers(0, cfg.vocab, 16).astype(np.int32)
        tok = dec.prefill(prompt)
        ref, alt = oracle.forward(prompt, 0)
        errs = [check_step("prefill", dec.logits_host(), tok, ref, alt)]
        dec.begin_decode(tok)
        pos = prompt.size
        for step in range(10):
            fed = tok
            tok = dec.decode_step()
            ref, alt = oracle.forward(np.array([fed], np.int32), pos)
            errs.append(check_step("decode %d" % step, dec.logits_host(), tok, ref, alt))
            pos += 1
        gpu_worst, self_worst = max(e for e, _ in errs), max(s_ for _, s_ in errs)
        gpu_mean, self_mean = float(np.mean([e for e, _ in errs])), float(np.mean([s_ for _, s_ in errs]))
        say("  worst/mean gpu: %.2e / %.2e   worst/mean cpu self-sensitivity: %.2e / %.2e" % (gpu_worst, gpu_mean, self_worst, self_mean))
        assert gpu_mean < 2 * self_mean + 1e-3
        assert gpu_worst < 3 * self_worst + 1e-3
    finally:
        dec.close()


def test_recorded_program_replays_equal_eager_steps(gpu, orc):
    # every replay is checked against the same step run eagerly, with eager work and
    # synchronisations between replays
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    w = SyntheticWeights(cfg, 3)
    a, b = Decoder(gpu, cfg, w), Decoder(gpu, cfg, w)
    try:
        prompt = np.random.default_rng(1).integers(0, cfg.vocab, 9).astype(np.int32)
        ta, tb = a.prefill(prompt), b.prefill(prompt)
        assert ta == tb
        a.begin_decode(ta)
        assert gpu.program_node_count(a.program) > 10
        for step in range(8):
            fed = ta
            ta = a.decode_step()                      # replayed graph
            la = a.logits_host()
            tb = b.decode_step_eager(fed)             # same step, launched eagerly
            lb = b.logits_host()
            gpu.sync()
            assert ta == tb, step
            assert np.array_equal(la, lb), step       # same kernels, same inputs: bit-identical
    finally:
        a.close(); b.close()


def test_decode_run_without_read_back_gives_the_same_tokens(gpu, orc):
    """A run of program replays with the loop state and the token log on the device (nothing read back between steps)
    against the same generation with a read-back after every step; then a second run continues where the first stopped."""
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    w = SyntheticWeights(cfg, 5)
    a, b = Decoder(gpu, cfg, w), Decoder(gpu, cfg, w)
    try:
        prompt = np.random.default_rng(2).integers(0, cfg.vocab, 7).astype(np.int32)
        ta, tb = a.prefill(prompt), b.prefill(prompt)
        assert ta == tb
        a.begin_decode(ta)
        b.begin_decode(tb)
        want = [b.decode_step() for _ in range(11)]
        got = list(a.decode_run(6)) + list(a.decode_run(5))
        assert got == want
    finally:
        a.close(); b.close()



@pytest.mark.parametrize("wdtype", [be.Q4_0, be.Q8_0])
def test_the_step_list_of_the_decoder_on_the_session_executor_gives_the_same_logits(gpu, wdtype):
    """The unfused step list (one record per graph step, in-place residual adds, workspace intermediates) run by the
    library's session executor against the hand-routed Decoder over the same weights: prefill and every replayed decode
    step give the same logits to the bit, and the executor folds a one-token layer into five calls."""
    from aion_amd.decoder import SessionDecoder
    cfg = DecoderConfig(wdtype=wdtype, **SMALL)
    w = SyntheticWeights(cfg, 7)
    a, b = Decoder(gpu, cfg, w), SessionDecoder(gpu, cfg, w)
    try:
        prompt = np.random.default_rng(4).integers(0, cfg.vocab, 11).astype(np.int32)
        ta, tb = a.prefill(prompt), b.prefill(prompt)
        assert np.array_equal(a.logits_host(), b.logits_host()) and ta == tb
        a.begin_decode(ta)
        b.begin_decode(tb)
        # per layer: q/k/v side, attention, o + add, feed-forward + add -> 4 calls; gather, head, argmax, copy, 3 adds around them
        assert b.calls_per_step == 4 * cfg.layers + 7
        for step in range(6):
            ta, tb = a.decode_step(), b.decode_step()
            assert np.array_equal(a.logits_host(), b.logits_host()), step
            assert ta == tb, step
        # a second prompt on the same objects: a longer prefill may replace a work buffer, the program is recorded again
        a.reset()
        b.pos = 0
        prompt = np.random.default_rng(5).integers(0, cfg.vocab, 40).astype(np.int32)
        ta, tb = a.prefill(prompt), b.prefill(prompt)
        assert np.array_equal(a.logits_host(), b.logits_host())
        a.begin_decode(ta)
        b.begin_decode(tb)
        for step in range(3):
            assert a.decode_step() == b.decode_step(), step
    finally:
        a.close(); b.close()
