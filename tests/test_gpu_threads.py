"""Calls from several host threads: the library serialises them (one lock around every exported function), so handles that
belong to different threads may be driven at the same time.  The reference's engine is single-session and its callers
serialise (neural/neuralchatengine.pas:58-60); its offload object gives every net one in-order queue
(examples/ChatTerminal/README.md:174-180).  Here the equivalent promise is tested: results under contention are bit-identical
to the results of the same calls made one after the other, and an error message stays with the thread whose call failed."""
import ctypes
import threading

import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.model_build import synthetic_spec

pytestmark = pytest.mark.gpu

CFG_A = dict(n_layers=2, d_model=512, n_q_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=1200, max_ctx=64, eps=1e-6, rope_theta=1e6)
CFG_B = dict(n_layers=3, d_model=256, n_q_heads=4, n_kv_heads=4, head_dim=64, ffn=512, vocab=700, max_ctx=64, eps=1e-5, rope_theta=1e4)
STEPS = 40


def greedy_with_logits(dec, first, steps):
    dec.reset(0)
    tok, toks, rows = first, [], []
    for p in range(steps):
        am, lg = dec.step(tok, p)
        rows.append(lg[0].copy()); tok = int(am[0]); toks.append(tok)
    return toks, np.array(rows)


def test_two_decoders_and_a_gemv_loop_on_three_threads_equal_the_serial_results():
    from helpers.device import dev
    cai = dev()
    dec_a = cai.Decoder(synthetic_spec(CFG_A, O.Q4_K, head_qtype=O.Q6_K, qkv_bias=True, std=0.05))
    dec_b = cai.Decoder(synthetic_spec(CFG_B, O.Q8_0, std=0.05))
    rng = np.random.default_rng(8)
    rows, cols = 333, 1024
    raw = O.quantize(O.Q4_K, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    w = cai.QWeight(O.Q4_K, rows, cols, raw)
    xs = rng.standard_normal((16, 1, cols)).astype(np.float32)

    serial_a = greedy_with_logits(dec_a, 5, STEPS)
    serial_b = greedy_with_logits(dec_b, 9, STEPS)
    serial_w = [w.gemv(x).copy() for x in xs]

    out, errors = {}, []
    gate = threading.Barrier(3)

    def run(name, fn):
        try:
            gate.wait()
            out[name] = fn()
        except Exception as e:                      # a failure in a worker must fail the test, not vanish with the thread
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=run, args=("a", lambda: greedy_with_logits(dec_a, 5, STEPS))),
               threading.Thread(target=run, args=("b", lambda: greedy_with_logits(dec_b, 9, STEPS))),
               threading.Thread(target=run, args=("w", lambda: [w.gemv(x).copy() for _ in range(6) for x in xs]))]
    for t in threads: t.start()
    for t in threads: t.join(120)
    assert not errors, errors
    assert not any(t.is_alive() for t in threads)
    assert out["a"][0] == serial_a[0] and np.array_equal(out["a"][1], serial_a[1])
    assert out["b"][0] == serial_b[0] and np.array_equal(out["b"][1], serial_b[1])
    for i, y in enumerate(out["w"]):
        assert np.array_equal(y, serial_w[i % len(xs)])
    w.close()


def test_an_error_message_stays_with_the_thread_whose_call_failed():
    from helpers.device import dev
    cai = dev()
    lib = cai.load()

    def last_error():
        buf = ctypes.create_string_buffer(512)
        lib.cai_last_error(buf, 512)
        return buf.value.decode()

    seen = {}

    def failing():
        rc = lib.cai_rope(None, 1, 64, 0, 1e4, 0)
        seen["rc"] = rc; seen["failing"] = last_error()

    def innocent():
        seen["innocent"] = last_error()

    t = threading.Thread(target=failing); t.start(); t.join(30)
    t = threading.Thread(target=innocent); t.start(); t.join(30)
    assert seen["rc"] != 0 and "cai_rope" in seen["failing"]
    assert seen["innocent"] == ""
