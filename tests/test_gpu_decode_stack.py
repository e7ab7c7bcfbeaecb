"""The one-launch decoder stack (aionhip_step_decoder_stack) against the launch-per-step schedule of the same decoder:
every phase calls the device functions of the separate steps in the same order per output, so over a cache of at most
256 tokens the two give the same bits - logits and greedy tokens compared exactly, step by step."""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip
from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


MID = dict(layers=3, hidden=2048, heads=8, kv_heads=1, head_dim=256, ffn=8192, vocab=8192, max_seq=96)
SMALL128 = dict(layers=2, hidden=1024, heads=8, kv_heads=2, head_dim=128, ffn=2048, vocab=4096, max_seq=64)


@pytest.mark.parametrize("shape,wdtype", [(MID, be.Q4_0), (MID, be.Q8_0), (SMALL128, be.Q4_0)])
def test_one_launch_stack_gives_the_bits_of_the_separate_steps(gpu, shape, wdtype):
    cfg = DecoderConfig(wdtype=wdtype, **shape)
    say("stack vs steps", shape, wdtype)
    weights = SyntheticWeights(cfg, seed=11)
    one = Decoder(gpu, cfg, weights, one_launch=True)
    ref = Decoder(gpu, cfg, weights, one_launch=False)
    try:
        assert one.stack is not None and ref.stack is None
        prompt = np.random.default_rng(5).integers(0, cfg.vocab, cfg.max_seq - 36).astype(np.int32)
        t_one, t_ref = one.prefill(prompt), ref.prefill(prompt)
        assert t_one == t_ref
        one.begin_decode(t_one)
        ref.begin_decode(t_ref)
        for step in range(24):
            say("  step", step)
            a, b = one.decode_step(), ref.decode_step()
            assert gpu.last_kernel() != ""
            la, lb = one.logits_host(), ref.logits_host()
            assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)), (step, float(np.abs(la - lb).max()))
            assert a == b
        gpu.decoder_stack_status(one.stack)
        # a run without read-backs gives the same tokens as the other schedule's
        assert np.array_equal(one.decode_run(8), ref.decode_run(8))
    finally:
        one.close()
        ref.close()


def test_a_stack_that_gives_up_waiting_reports_it_and_recovers(gpu):
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL128)
    weights = SyntheticWeights(cfg, seed=3)
    one = Decoder(gpu, cfg, weights, one_launch=True)
    ref = Decoder(gpu, cfg, weights, one_launch=False)
    try:
        prompt = np.arange(10, dtype=np.int32)
        t = one.prefill(prompt)
        assert ref.prefill(prompt) == t
        one.begin_decode(t)
        ref.begin_decode(t)
        gpu.decoder_stack_set_poll_budget(one.stack, 0)          # every workgroup leaves at its first unanswered poll
        say("  forcing the give-up path")
        one._forward(1, one._decode_buffers)
        with pytest.raises(be.AionHipError) as e:
            gpu.decoder_stack_status(one.stack)
        assert e.value.status == hip.EXECUTION_FAILED
        gpu.decoder_stack_set_poll_budget(one.stack, 250)
        say("  and again with the normal budget")
        one._set_decode_state(one._decode_buffers, t, one.pos)     # same step again: the caches rows are rewritten with the same values
        a, b = one.decode_step(), ref.decode_step()
        gpu.decoder_stack_status(one.stack)
        assert a == b and np.array_equal(one.logits_host().view(np.uint32), ref.logits_host().view(np.uint32))
    finally:
        one.close()
        ref.close()


def test_stack_refuses_shapes_outside_its_limits(gpu):
    cfg = DecoderConfig(layers=1, hidden=512, heads=8, kv_heads=1, head_dim=64, ffn=1024, vocab=2048, max_seq=48)
    dec = Decoder(gpu, cfg, SyntheticWeights(cfg, seed=1), one_launch=True)
    try:
        assert dec.stack is None                                 # head size 64: separate steps
        t = dec.prefill(np.arange(5, dtype=np.int32))
        dec.begin_decode(t)
        dec.decode_step()
    finally:
        dec.close()
