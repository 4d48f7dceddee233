"""Width-K window steps and prompt-lookup generation on the device session.

The reference's contract (neural/neuraldecode.pas:1151-1183, 5696-5712): a width-K StepForward at absolute position p gives, row
by row, what K width-1 steps at p, p+1, ... give, and TruncateTo rolls the cache back over the rows the caller does not commit
(examples/SpeculativeDecoding/SpeculativeDecoding.lpr:646-663, 806-810).  DecodePromptLookup's gates
(tests/TestNeuralDecode.pas:1573-1631): the text equals plain greedy decoding for (MatchLen, NumDraft) = (2, 3) and (3, 5) on a
repetitive prompt, and a MatchLen longer than the context degrades to one token per pass."""
import numpy as np
import pytest

from helpers import oracle_lib as O
from helpers.model_build import oracle_model, synthetic_spec
from test_gpu_decoder import SHAPES

pytestmark = pytest.mark.gpu


def make(name, **kw):
    from helpers.device import dev
    cai = dev()
    s = SHAPES[name]
    spec = synthetic_spec(s["cfg"], s["qtype"], head_qtype=s["head"], qkv_bias=s["bias"], std=0.05)
    return cai, spec, cai.Decoder(spec, **kw)


@pytest.mark.parametrize("name", ["qwen7b_like_q4k", "smollm_like_q8", "llama_like_q4_0", "olmoe_like_q8", "llama_like_q6k"])
@pytest.mark.parametrize("kv", ["f32", "f16"])
def test_window_rows_equal_single_steps_and_the_oracle(name, kv):
    from helpers.device import rel_err
    cai, spec, dec = make(name, kv_dtype={"f32": 0, "f16": 1}[kv])     # max_batch 1: a window needs no second sequence
    rng = np.random.default_rng(11)
    toks = rng.integers(0, spec["cfg"]["vocab"], 40).tolist()
    om = oracle_model(spec, acc64=1, kv_f16=1 if kv == "f16" else 0)
    ref = [om.step(t, p)[1] for p, t in enumerate(toks)]
    single = [dec.step(t, p)[1][0].copy() for p, t in enumerate(toks)]
    worst_o, worst_s = 0.0, 0.0
    for n in (2, 3, 5, 8):
        dec.truncate(12)
        am, lg = dec.step_window(toks[12:12 + n], 12)
        assert dec.len() == 12 + n
        for r in range(n):
            worst_o = max(worst_o, rel_err(lg[r], ref[12 + r])); worst_s = max(worst_s, rel_err(lg[r], single[12 + r]))
            assert int(am[r]) == int(np.argmax(lg[r]))
        # commit three rows of the window (or all of a narrower one), drop the rest, go on token by token: the kept rows are the right ones
        keep = min(n, 3)
        dec.truncate(12 + keep)
        _, l1 = dec.step(toks[12 + keep], 12 + keep)
        worst_s = max(worst_s, rel_err(l1[0], single[12 + keep]))
    assert worst_o < 1e-3, worst_o       # the north-star logits tolerance, against the float64-accumulating oracle
    assert worst_s < 2e-4, worst_s       # against the device's own width-1 steps (other kernels, same arithmetic up to summation order)
    # width 1 is a plain step
    dec.truncate(12)
    am, lg = dec.step_window([toks[12]], 12)
    assert np.array_equal(lg[0], single[12])


def test_window_on_another_sequence_and_over_an_int8_cache():
    from helpers.device import rel_err
    cai, spec, dec = make("qwen7b_like_q4k", max_batch=3, kv_dtype=2)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, spec["cfg"]["vocab"], 30).tolist()
    dec.prefill(toks[:10], 0, seq=2, want_logits=False)
    single = []
    for i in range(8):
        single.append(dec.step_window([toks[10 + i]], 10 + i, seq=2)[1][0].copy())
    dec.truncate(10, seq=2)
    am, lg = dec.step_window(toks[10:18], 10, seq=2)
    assert dec.len(2) == 18 and dec.len(0) == 0
    # (rows of an int8 cache are quantised when they are appended: both paths quantise the same rows)
    assert max(rel_err(lg[r], single[r]) for r in range(8)) < 2e-3


def simulate_lookup(context, greedy, match_len, num_draft, n):
    """passes the lookup loop takes when the model's outputs are the known greedy continuation `greedy`"""
    all_t, emitted, passes = list(context), 0, 0
    while emitted < n:
        room = min(num_draft, 7, n - emitted - 1)
        draft = O.prompt_lookup_draft(all_t, match_len, room) if room > 0 else []
        passes += 1
        all_t.append(greedy[emitted]); emitted += 1
        acc = 0
        while acc < len(draft) and emitted < n and draft[acc] == greedy[emitted - 1]:
            acc += 1; all_t.append(greedy[emitted]); emitted += 1
    return passes


@pytest.mark.parametrize("name", ["qwen7b_like_q4k", "smollm_like_q8", "olmoe_like_q8"])
def test_lookup_generation_equals_greedy_and_takes_the_predicted_passes(name):
    cai, spec, dec = make(name)
    prompt = [7, 11, 13] * 4                               # 'abcabcabcabc'
    n = 64
    dec.prefill(prompt[:-1], 0, want_logits=False)
    greedy = dec.generate(prompt[-1], len(prompt) - 1, n).tolist()
    assert dec.len() == len(prompt) - 1 + n
    took = {}
    for match_len, num_draft in ((2, 3), (3, 5), (1, 7), (64, 4)):
        dec.truncate(len(prompt) - 1)
        got, passes = dec.generate_lookup(prompt, n, match_len, num_draft)
        assert got.tolist() == greedy, (match_len, num_draft)
        assert dec.len() == len(prompt) - 1 + n
        assert passes == simulate_lookup(prompt, greedy, match_len, num_draft, n), (match_len, num_draft)
        took[(match_len, num_draft)] = passes
    assert took[(64, 4)] == n                              # no earlier occurrence can exist: one token per pass
    # and the session continues from there like after plain generation
    nxt = dec.step(greedy[-1], dec.len(), want_logits=False)[0]
    dec.truncate(len(prompt) - 1)
    assert dec.generate(prompt[-1], len(prompt) - 1, n + 1).tolist()[-1] == int(nxt[0])


def test_a_draft_of_the_true_continuation_is_accepted_whole():
    cai, spec, dec = make("qwen7b_like_q4k")
    dec.prefill([3, 1, 4, 1, 5, 9, 2, 6], 0, want_logits=False)
    g = dec.generate(5, 8, 9).tolist()
    dec.truncate(8)
    am, _ = dec.step_window([5] + g[:7], 8, want_logits=False)
    assert am.tolist() == g[:8]


def test_window_and_lookup_refusals():
    cai, spec, dec = make("llama_like_q4_0")
    with pytest.raises(cai.CaiError, match="width 9"):
        dec.step_window(list(range(9)), 0)
    with pytest.raises(cai.CaiError, match="is at position 0"):
        dec.step_window([1, 2], 5)
    with pytest.raises(cai.CaiError, match="outside vocab"):
        dec.step_window([1, spec["cfg"]["vocab"]], 0)
    with pytest.raises(cai.CaiError, match="exceed max_ctx"):
        dec.prefill(list(range(90)), 0, want_logits=False); dec.step_window([1] * 8, 90)
    dec.reset()
    with pytest.raises(cai.CaiError, match="holds 0 tokens"):
        dec.generate_lookup([1, 2, 3], 4)
    with pytest.raises(cai.CaiError, match="exceed max_ctx"):
        dec.generate_lookup([1], 97)
    dec.set_eviction(4, 32)
    dec.step_window([1], 0)                                   # one token at a time still works
    with pytest.raises(cai.CaiError, match="eviction"):
        dec.step_window([1, 2], 1)
    out, passes = dec.generate_lookup([1, 1], 12, 1, 4)       # drafts are switched off: one token per pass
    assert passes == 12 and len(out) == 12
    # and, like plain generation, the rolling session runs past max_ctx
    dec.reset(); dec.step_window([1], 0)
    plain = dec.generate(1, 1, 96).tolist()
    dec.reset(); dec.step_window([1], 0)
    out, passes = dec.generate_lookup([1, 1], 96, 1, 4)
    assert out.tolist() == plain and passes == 96 and dec.len() == 97


@pytest.mark.parametrize("name", ["qwen7b_like_q4k", "smollm_like_q8", "olmoe_like_q8"])
def test_hidden_state_after_steps_windows_prompts_and_generation(name):
    """HiddenState of the reference session (neural/neuraldecode.pas:1314-1321, 5850-5857): the vector the vocabulary projection reads.
    Pinned two ways: against the oracle's final-norm output at the same position (1e-4 of its largest element), and through the
    head itself - projecting the returned vector with the oracle's head product gives the step's logits."""
    from helpers.device import rel_err
    cai, spec, dec = make(name)
    rng = np.random.default_rng(21)
    toks = rng.integers(0, spec["cfg"]["vocab"], 24).tolist()
    om = oracle_model(spec, acc64=1)
    hid = []
    for p, t in enumerate(toks):
        om.step(t, p); hid.append(om.hidden())
        _, lg = dec.step(t, p)
        if p in (0, 7, 23):
            h = dec.hidden_state()
            assert rel_err(h, hid[p]) < 1e-4, p
            head = spec["tensors"].get((-1, O.W_HEAD)) or spec["tensors"][(-1, O.W_EMBED)]
            proj = O.gemv(head["type"], head["raw"], head["rows"], head["cols"], h[None, :], None, 0, 1)
            assert rel_err(proj[0], lg[0]) < 1e-4
    # rows of a window
    dec.truncate(10)
    dec.step_window(toks[10:16], 10, want_logits=False)
    for r in (0, 3, 5):
        assert rel_err(dec.hidden_state(r), hid[10 + r]) < 1e-4, r
    # after a prompt pass and after device-side generation: row 0 is the last token fed
    dec.reset(); dec.prefill(toks[:20], 0, want_logits=False)
    assert rel_err(dec.hidden_state(), hid[19]) < 1e-4
    g = dec.generate(toks[20], 20, 3)
    om.truncate(20); om.step(toks[20], 20); om.step(int(g[0]), 21); om.step(int(g[1]), 22)
    assert rel_err(dec.hidden_state(), om.hidden()) < 1e-4
    with pytest.raises(cai.CaiError, match="row 8"):
        dec.hidden_state(8)


@pytest.mark.parametrize("kv", [0, 2])
def test_forked_sequences_step_as_a_batch_like_sequences_built_one_by_one(kv):
    """The cache fork of a beam search (DecodeBeamSearchCachedAll, neural/neuraldecode.pas:1436-1453: every surviving hypothesis
    continues from its parent's cache): sequence 0 ingests the prompt, sequences 1..3 are forked from it - directly, and through a
    snapshot restored into another sequence -, then all four take DIFFERENT tokens in one batched step.  Each row must equal a
    session that ingested prompt + that token alone."""
    from helpers.device import rel_err
    cai, spec, dec = make("qwen7b_like_q4k", max_batch=4, kv_dtype=kv)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, spec["cfg"]["vocab"], 20).tolist()
    branch = [[5, 9], [17, 3], [900, 41], [2, 2]]
    want = []
    for b in range(4):
        dec.reset(0); dec.prefill(prompt, 0, want_logits=False)
        dec.step(branch[b][0], 20, want_logits=False)
        want.append(dec.step(branch[b][1], 21)[1][0].copy())
    dec.reset(0); dec.prefill(prompt, 0, want_logits=False)
    dec.fork(0, 1); dec.fork(0, 2)
    snap = dec.snapshot(0); dec.restore(snap, seq=3); cai.load().cai_kv_snap_destroy(snap)
    assert [dec.len(b) for b in range(4)] == [20] * 4
    dec.step([br[0] for br in branch], [20] * 4, want_logits=False)
    _, lg = dec.step([br[1] for br in branch], [21] * 4)
    for b in range(4):
        assert rel_err(lg[b], want[b]) < (2e-3 if kv == 2 else 2e-4), b
    # a fork overwrites what the target held, and a fork onto itself is a no-op
    dec.fork(1, 0); dec.fork(2, 2)
    assert dec.len(0) == 22
    _, l0 = dec.step([7], [22])
    dec.truncate(22, seq=1)
    dec.reset(0); dec.prefill(prompt + branch[1], 0, want_logits=False)
    _, l1 = dec.step([7], [22])
    assert rel_err(l0[0], l1[0]) < (2e-3 if kv == 2 else 2e-4)
    with pytest.raises(cai.CaiError, match="sequences 0 -> 4"):
        dec.fork(0, 4)
