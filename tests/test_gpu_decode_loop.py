"""The decode loop's glue around the draws (src/generate.rs:776-891, src/qwen4exp/batch.rs:138-162):
ping-pong output slots read through polled completion, the next step enqueued while the current
one runs, and a sequence's counts handed from the engine's scratch to a batch slot and back."""
import numpy as np
import pytest
import torch

import lily_sampler as LS
import oracle as O
from gpu_util import dev, ls_params, o_params

pytestmark = pytest.mark.gpu

# tests/test_batch.rs / tests/unit/kernels/sample.rs: the reference's SAMPLED request
SAMPLED = dict(temperature=1.0, top_k=20, top_p=0.95, presence_penalty=1.5, seed=7)


def _model(rng, vocab, contexts):
    """A stand-in for the model: the logits a step sees depend on the token before it."""
    return rng.normal(0, 2.5, (contexts, vocab)).astype(np.float32)


def _oracle_sequence(table, first, steps, op, counts):
    toks, tok = [], first
    for t in range(steps):
        d = O.sample(table[tok % len(table)], counts, op, t)
        tok = int(d.chosen)
        counts[tok] += 1
        toks.append(tok)
    return toks


@pytest.mark.parametrize("ahead", [False, True], ids=["serial", "next-step-in-flight"])
def test_two_steps_in_flight_draw_what_serial_steps_draw(ahead):
    s = LS.Sampler(0)
    rng = np.random.default_rng(3)
    vocab, contexts, steps, first = 40_009, 16, 40, 123
    table = _model(rng, vocab, contexts)
    t_table = torch.from_numpy(table).to(dev())
    lp, op = ls_params(**SAMPLED), o_params(**SAMPLED)
    scratch = LS.SamplerScratch(s, vocab)
    slots = LS.TokenSlots(s, slots=2, words=1)
    row = torch.zeros(1, dtype=torch.int32, device=dev())
    slots.device(0).fill_(first)          # the prefill's draw sits in slot 0
    torch.cuda.synchronize()

    def enqueue(step, slot_in, slot_out):
        # "the model": which logits the step sees follows from the token in slot_in, on the device
        torch.remainder(slots.device(slot_in), contexts, out=row)
        s.sample_f32_at(t_table, row, scratch, lp, step, None, slots.device(slot_out))
        slots.publish(slot_out)

    got, slot_in = [], 0
    if ahead:
        enqueue(0, 0, 1)
        for t in range(steps):
            if t + 1 < steps:
                # the following step reads the slot this one writes; it is on the stream before the
                # host has seen this step's token
                enqueue(t + 1, 1 - slot_in, slot_in)
            got.append(slots.wait_polled(1 - slot_in)[0])
            slot_in = 1 - slot_in
    else:
        for t in range(steps):
            enqueue(t, slot_in, 1 - slot_in)
            s.synchronize()
            words = slots.poll(1 - slot_in)
            assert words is not None       # the stream has drained: the poll must see it
            got.append(words[0])
            slot_in = 1 - slot_in
    want = _oracle_sequence(table, first, steps, op, np.zeros(vocab, np.uint32))
    assert got == want
    assert len(set(got)) > 5               # the sequence moves through the contexts
    slots.close()
    scratch.close()
    s.close()


def test_poll_does_not_block_and_slots_must_be_read_in_turn():
    s = LS.Sampler(0)
    slots = LS.TokenSlots(s, slots=2, words=3)
    with pytest.raises(LS.SamplerError):
        slots.poll(0)                      # nothing published yet
    slots.device(1).copy_(torch.tensor([7, 8, 9], dtype=torch.int32))
    slots.publish(1)
    assert slots.wait_polled(1, max_polls=10_000_000) == [7, 8, 9]
    with pytest.raises(LS.SamplerError):
        slots.poll(1)                      # read already
    slots.close()
    s.close()


def test_a_sequence_moved_into_a_batch_slot_and_back_draws_what_it_draws_alone():
    """Engine scratch -> batch slot -> engine scratch (move_sampler_counts): the sequence's draws
    are those of the same sequence decoded alone, whatever shares its launches."""
    s = LS.Sampler(0)
    rng = np.random.default_rng(12)
    vocab, contexts, first = 40_009, 16, 77
    table = _model(rng, vocab, contexts)
    others = rng.normal(0, 2.5, (3, vocab)).astype(np.float32)
    t_table = torch.from_numpy(table).to(dev())
    lp, op = ls_params(**SAMPLED), o_params(**SAMPLED)
    engine = LS.SamplerScratch(s, vocab)
    batch = [LS.SamplerScratch(s, vocab) for _ in range(4)]
    out1 = torch.zeros(1, dtype=torch.int32, device=dev())
    out4 = torch.zeros(4, dtype=torch.int32, device=dev())
    got, tok = [], first
    for t in range(30):
        phase = (t // 6) % 2               # six steps alone, six steps as row 2 of a batch of four
        if t % 6 == 0 and t > 0:
            if phase == 1:
                engine.move_counts_to(batch[2])
            else:
                batch[2].move_counts_to(engine)
        if phase == 0:
            s.sample_f32(t_table[tok % contexts], engine, lp, t, out1)
            s.synchronize()
            tok = int(out1.cpu()[0])
        else:
            rows = np.stack([others[0], others[1], table[tok % contexts], others[2]])
            params = [ls_params(**dict(SAMPLED, seed=100 + r)) for r in range(4)]
            params[2] = lp
            s.sample_rows(torch.from_numpy(rows).to(dev()), params, [t] * 4, out4, scratch=batch)
            s.synchronize()
            tok = int(out4.cpu()[2])
        got.append(tok)
    want = _oracle_sequence(table, first, 30, op, np.zeros(vocab, np.uint32))
    assert got == want
    engine.move_counts_to(engine)          # from == to: nothing happens
    for x in batch + [engine]:
        x.close()
    s.close()


def test_insertions_keep_the_counts_the_oracle_keeps():
    """The thinking control's answers as forced tokens (src/thinking.rs:485-608), with the
    replaced draw taken out of the penalty counts (the TODO at thinking.rs:587-592).  Two rows
    decode under SAMPLED; at step 2 row 0's draw is replaced by three ids, at step 3 row 1 gets
    two ids in front of its draw.  Every token equals the oracle's on the same counts, and the
    counts at the end hold exactly the tokens that were emitted."""
    sampler = LS.Sampler(0)
    rng = np.random.default_rng(31)
    rows, steps_n, VOCAB = 2, 9, 30_011
    x = rng.normal(0.0, 2.0, (steps_n, rows, VOCAB)).astype(np.float32)
    sc = [LS.SamplerScratch(sampler, VOCAB) for _ in range(rows)]
    counts = [np.zeros(VOCAB, dtype=np.uint32) for _ in range(rows)]
    q = LS.Insertions(rows)
    params = [LS.SamplingParams.greedy(**dict(SAMPLED, seed=7 + r)) for r in range(rows)]
    oparams = [O.params(**dict(SAMPLED, seed=7 + r)) for r in range(rows)]
    out = torch.zeros(rows, dtype=torch.int32, device=dev())
    emitted = [[] for _ in range(rows)]
    replace_ids, before_ids = [VOCAB - 1, 17, 17], [5, 6]
    for step in range(steps_n):
        forced, _ = q.next()
        logits = torch.from_numpy(x[step]).to(dev())
        keep = sampler.sample_rows(logits, params, [step] * rows, out, scratch=sc, forced=forced)
        sampler.synchronize()
        del keep
        got = out.cpu().numpy()
        for r in range(rows):
            d = O.sample(x[step, r], counts[r], oparams[r], step, forced=forced[r])
            assert got[r] == d.chosen, (step, r)
            if forced[r] is not None:
                assert got[r] == forced[r]
            emitted[r].append(int(got[r]))
        if step == 2:     # row 0: the draw was a stop token; the close replaces it
            q.push(0, LS.INSERT_REPLACE, drawn=int(got[0]), ids=replace_ids, scratch=sc[0])
            counts[0][got[0]] -= 1
            emitted[0].pop()
        if step == 3:     # row 1: a close tag in front of the tool call just drawn
            q.push(1, LS.INSERT_BEFORE, drawn=int(got[1]), ids=before_ids, scratch=sc[1])
            counts[1][got[1]] -= 1
            drawn_again = emitted[1].pop()
        if step == 6:
            assert emitted[1][5] == drawn_again   # ... which followed the two inserted ids
    for r in range(rows):
        assert np.array_equal(sc[r].read_counts().numpy().view(np.uint32), counts[r]), r
        assert np.array_equal(np.bincount(emitted[r], minlength=VOCAB).astype(np.uint32), counts[r]), r
    assert emitted[0][2:5] == replace_ids
    assert emitted[1][3:5] == before_ids
    q.close()
    for s_ in sc:
        s_.close()
    sampler.close()
