"""GPU parity: the device sampler and the batched generation loop vs the oracle's restatement of
src/module/sample.rs and of GpuMambaLM::generate_batch / generate (src/module/gpu_lm.rs:323-516).

Bar: the generator state is integer work and must match bit for bit.  A sampled token is an index picked by
comparing a draw r with running sums of probabilities; the device forms those sums as f64 tree sums, the
reference as sequential f32 sums (and its exp is the Cephes polynomial, SIMD-dependent), so a token may differ
only when r lies within 2e-5 of the boundary between the two tokens in the oracle's own distribution -- checked
case by case below, with the number of such cases bounded.
"""
import numpy as np
import pytest
import torch

import orc
from test_engine_gpu import oracle_params

from mamba_rs_amd import GpuMambaBackbone, GpuMambaLM, MambaConfig, MambaWeights, SampleParams, ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SLACK = 2e-5


def device_sample(logits, params_rows, seeds, seen_lists=None, active=None):
    rows, vocab = logits.shape
    sp = np.array([[p.temperature, p.top_k, p.top_p, p.min_p, p.repetition_penalty] for p in params_rows], np.float32)
    state = np.array([ops.xoshiro_seed(s) for s in seeds], dtype=np.uint64).view(np.int64)
    rng = torch.from_numpy(state).to(DEV)
    seen = None
    if seen_lists is not None:
        cnt = np.zeros((rows, vocab), np.int32)
        for r, lst in enumerate(seen_lists):
            for t in lst:
                if t < vocab:
                    cnt[r, t] += 1
        seen = torch.from_numpy(cnt).to(DEV)
    act = None if active is None else torch.tensor(active, dtype=torch.int32, device=DEV)
    tok = ops.sample_tokens(torch.from_numpy(logits).to(DEV), sp, rng, seen_counts=seen, active=act)
    torch.cuda.synchronize()
    return tok.cpu().numpy(), rng.cpu().numpy().view(np.uint64)


def check_row(got, logits_row, p: SampleParams, seed, seen=()):
    """-> 0 if the token equals the oracle's, 1 if it differs within the boundary slack; asserts otherwise."""
    g = orc.Xoshiro(seed=seed)
    want, probs = orc.sample_token(logits_row, g, p.temperature, p.top_k, p.top_p, p.min_p, p.repetition_penalty, seen)
    if got == want:
        return 0, g.state()
    assert p.temperature > 0, f"greedy pick {got} != {want}"
    r = orc.Xoshiro(seed=seed).next_f32()
    cum = np.cumsum(probs.astype(np.float64))
    lo = cum[got - 1] if got > 0 else 0.0
    assert probs[got] > 0 or abs(r - lo) < SLACK, f"token {got} has no mass in the oracle's distribution (oracle picked {want})"
    assert lo - SLACK <= r < cum[got] + SLACK, f"token {got}: draw {r} outside [{lo}, {cum[got]}) by more than the slack (oracle {want})"
    return 1, g.state()


CASES = [
    SampleParams(temperature=1.0),
    SampleParams(temperature=0.7),
    SampleParams(temperature=1.3, top_k=50),
    SampleParams(temperature=0.8, top_k=1),
    SampleParams(temperature=1.0, top_p=0.9),
    SampleParams(temperature=0.9, top_k=200, top_p=0.8),
    SampleParams(temperature=1.0, min_p=0.05),
    SampleParams(temperature=0.8, top_k=40, top_p=0.95, min_p=0.02, repetition_penalty=1.3),
    SampleParams(temperature=1.0, top_p=0.3, repetition_penalty=0.8),
    SampleParams(temperature=0.0),
    SampleParams(temperature=0.0, repetition_penalty=1.5),
    SampleParams(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, repetition_penalty=float("nan")),
]


@pytest.mark.parametrize("vocab,scale", [(50280, 2.5), (1000, 4.0), (77, 1.0)])
def test_sampler_rows_match_the_oracle(vocab, scale):
    rng = np.random.default_rng(vocab)
    rows = len(CASES) * 6
    params = [CASES[r % len(CASES)] for r in range(rows)]
    # a handful of distinct logit rows (a peaked one among them), each row its own seed and seen list
    base = (rng.standard_normal((4, vocab)) * scale).astype(np.float32)
    base[3] *= 3.0
    logits = np.stack([base[r % 4] for r in range(rows)])
    seeds = [1000 + 7 * r for r in range(rows)]
    seen = [list(rng.integers(0, vocab, 20)) + [int(np.argmax(logits[r]))] * 2 for r in range(rows)]
    tok, state = device_sample(logits, params, seeds, seen)
    near = 0
    for r in range(rows):
        d, want_state = check_row(int(tok[r]), logits[r], params[r], seeds[r], seen[r])
        near += d
        assert [int(v) for v in state[r]] == want_state, f"row {r}: generator state"
    assert near <= 1, f"{near} of {rows} rows differ from the oracle (each within the boundary slack)"


def test_many_draws_stay_inside_the_filtered_support_and_follow_the_distribution():
    vocab, rows = 5000, 1024
    rng = np.random.default_rng(1)
    row = (rng.standard_normal(vocab) * 3).astype(np.float32)
    p = SampleParams(temperature=0.9, top_k=30, top_p=0.9)
    logits = np.tile(row, (rows, 1))
    seeds = list(range(5000, 5000 + rows))
    tok, _ = device_sample(logits, [p] * rows, seeds)
    _, probs = orc.sample_token(row, orc.Xoshiro(seed=0), p.temperature, p.top_k, p.top_p)
    support = np.flatnonzero(probs > 0)
    assert 1 < support.size <= 30 and set(tok.tolist()) <= set(support.tolist())
    near = sum(check_row(int(tok[r]), row, p, seeds[r])[0] for r in range(0, rows, 8))
    assert near <= 1
    freq = np.bincount(tok, minlength=vocab)[support] / rows
    assert np.abs(freq - probs[support]).max() < 0.05


def test_ties_keep_the_lower_index_and_greedy_keeps_the_last_maximum():
    vocab = 4096
    rng = np.random.default_rng(2)
    row = np.round(rng.standard_normal(vocab) * 2).astype(np.float32) / 2     # heavily tied values
    for p in (SampleParams(temperature=1.0, top_k=100), SampleParams(temperature=1.0, top_p=0.5), SampleParams(temperature=1.0, top_k=300, top_p=0.7)):
        rows = 256
        seeds = list(range(rows))
        tok, _ = device_sample(np.tile(row, (rows, 1)), [p] * rows, seeds)
        _, probs = orc.sample_token(row, orc.Xoshiro(seed=0), p.temperature, p.top_k, p.top_p)
        assert set(tok.tolist()) <= set(np.flatnonzero(probs > 0).tolist())
        assert sum(check_row(int(tok[r]), row, p, seeds[r])[0] for r in range(rows)) <= 1
    flat = np.zeros((2, vocab), np.float32); flat[1, 5] = flat[1, 900] = 3.0
    tok, state = device_sample(flat, [SampleParams(temperature=0.0)] * 2, [1, 2])
    assert tok.tolist() == [vocab - 1, 900]
    assert [int(v) for v in state[0]] == ops.xoshiro_seed(1)       # the greedy branch draws nothing


def test_inactive_rows_are_left_alone():
    vocab = 300
    logits = np.random.default_rng(3).standard_normal((4, vocab)).astype(np.float32)
    tok, state = device_sample(logits, [SampleParams()] * 4, [1, 2, 3, 4], active=[1, 0, 1, 0])
    assert tok[1] == -1 and tok[3] == -1 and tok[0] >= 0 and tok[2] >= 0
    assert [int(v) for v in state[1]] == ops.xoshiro_seed(2) and [int(v) for v in state[0]] != ops.xoshiro_seed(1)


# ---- generation loops ---------------------------------------------------------------------------------

def oracle_generate_batch(P, embed, table, prompts, params, seen_includes_prompt=False):
    """generate_batch of src/module/gpu_lm.rs:389-516 (and, for one slot with seen_includes_prompt, the same tokens as
    generate_streaming, :334-377) on the oracle's backbone: -> (tokens per slot, per-token records for tolerance checks)."""
    B = len(prompts)
    states = [orc.m1_zero_state(P) for _ in range(B)]
    rngs = [orc.Xoshiro(seed=p.seed) for p in params]
    pos, finished = [0] * B, [False] * B
    outputs, last = [[] for _ in range(B)], [0] * B
    records = [[] for _ in range(B)]
    for i in range(B):
        if len(prompts[i]) == 0:
            finished[i] = True
        else:
            last[i], pos[i] = prompts[i][0], 1
    total = max(len(p) for p in prompts) + max(p.max_tokens for p in params)
    for _ in range(total):
        if all(finished):
            break
        for i in range(B):
            if finished[i]:
                continue
            conv, ssm = states[i]
            h = orc.m1_backbone_step(P, embed[last[i]], conv, ssm, identity_proj=True)
            if pos[i] < len(prompts[i]):
                last[i] = prompts[i][pos[i]]; pos[i] += 1
                continue
            logits = (table @ h).astype(np.float32)
            sp = params[i]
            seen = (list(prompts[i]) if seen_includes_prompt else []) + outputs[i]
            r = orc.Xoshiro(state=rngs[i].state()).next_f32()
            nxt, probs = orc.sample_token(logits, rngs[i], sp.temperature, sp.top_k, sp.top_p, sp.min_p, sp.repetition_penalty, seen)
            if nxt in sp.eos_token_ids or len(outputs[i]) >= sp.max_tokens:
                finished[i] = True
                continue
            records[i].append((nxt, probs, r, logits))
            outputs[i].append(nxt); last[i] = nxt
    return outputs, records


def assert_follows(got, want, records, params):
    """Tokens equal the oracle's up to the first position where the oracle's own pick sits on a boundary."""
    for i, (g, w) in enumerate(zip(got, want)):
        for j, (a, b) in enumerate(zip(g, w)):
            if a == b:
                continue
            nxt, probs, r, logits = records[i][j]
            if params[i].temperature <= 0:
                top = np.sort(logits)[-2:]
                assert top[1] - top[0] < 1e-3, f"slot {i} token {j}: greedy {a} != {b}"
            else:
                cum = np.cumsum(probs.astype(np.float64))
                lo = cum[a - 1] if a > 0 else 0.0
                assert lo - 1e-4 <= r < cum[a] + 1e-4, f"slot {i} token {j}: {a} != {b} away from a boundary"
            break
        else:
            assert len(g) == len(w), f"slot {i}: {len(g)} tokens, oracle {len(w)}"


def small_lm(batch, untied=False):
    cfg = MambaConfig(d_model=64, d_state=16, d_conv=4, expand=2, n_layers=2)
    w = MambaWeights.random_lm(cfg, seed=5, std=0.1)
    rng = np.random.default_rng(6)
    vocab = 300
    embed = (rng.standard_normal((vocab, 64)) * 0.5).astype(np.float32)
    head = (rng.standard_normal((64, vocab)) * 0.5).astype(np.float32) if untied else None
    eng = GpuMambaBackbone.new(0, w, cfg, 64, batch)
    return GpuMambaLM(eng, embed, head), oracle_params(w, cfg, 64), embed, (head.T if untied else embed)


def test_generate_batch_ragged_prompts_follow_the_oracle():
    lm, P, embed, table = small_lm(5)
    prompts = [[1, 2, 3, 250, 17, 9, 9], [], [42], [5, 6], [7, 8, 9, 10]]
    params = [SampleParams(temperature=0.0, max_tokens=10),
              SampleParams(max_tokens=4),
              SampleParams(temperature=8.0, top_k=20, max_tokens=12, seed=1),       # this tiny tied LM is peaked: high temperatures
              SampleParams(temperature=6.0, top_p=0.9, min_p=0.01, repetition_penalty=1.4, max_tokens=7, seed=2),
              SampleParams(temperature=6.0, max_tokens=40, seed=3)]
    free, _ = oracle_generate_batch(P, embed, table, prompts, params)
    assert len(set(free[4])) > 20 and len(set(free[2])) > 3, "the sampled slots should wander in this setup"
    params[4].eos_token_ids = [free[4][9]] + list(range(301, 316))           # ends slot 4 at its tenth token at the latest
    want, rec = oracle_generate_batch(P, embed, table, prompts, params)
    got = lm.generate_batch(prompts, params)
    assert got[1] == [] and len(got[0]) == 10 and len(got[2]) == 12 and len(got[3]) == 7
    assert len(want[4]) <= 9, "the EOS list should end slot 4 early in this setup"
    assert_follows(got, want, rec, params)
    # a second call on the same engine (replayed step graph, fresh state and generators) gives the same tokens
    assert lm.generate_batch(prompts, params) == got
    # other prompts / sizes on the same engine: buffers grow, the captured step stays valid
    prompts2 = [[3] * 40, [4, 5], [6], [7, 7, 7], [8]]
    params2 = [SampleParams(temperature=8.0, top_k=10, max_tokens=25, seed=10 + i) for i in range(5)]
    want2, rec2 = oracle_generate_batch(P, embed, table, prompts2, params2)
    assert_follows(lm.generate_batch(prompts2, params2), want2, rec2, params2)
    lm.close(); lm.backbone.close()


@pytest.mark.parametrize("untied", [False, True])
def test_generate_with_params_counts_the_prompt_as_seen(untied):
    lm, P, embed, table = small_lm(1, untied)
    prompt = [3, 3, 3, 17, 99]
    sp = SampleParams(temperature=6.0, top_k=30, repetition_penalty=1.8, max_tokens=16, seed=9, eos_token_ids=[299])
    want, rec = oracle_generate_batch(P, embed, table, [prompt], [sp], seen_includes_prompt=True)
    got = lm.generate(prompt, params=sp)
    assert_follows([got], want, rec, [sp])
    want_b, _ = oracle_generate_batch(P, embed, table, [prompt], [sp], seen_includes_prompt=False)
    assert want_b != want, "the penalty over the prompt should matter in this setup"
    # greedy through the sampled loop equals the greedy loop
    g = SampleParams(temperature=0.0, max_tokens=8)
    assert lm.generate(prompt, params=g) == lm.generate(prompt, 8)
    lm.close(); lm.backbone.close()


def test_generate_long_prompt_takes_the_prefill_route():
    lm, P, embed, table = small_lm(1)
    rng = np.random.default_rng(8)
    prompt = [int(t) for t in rng.integers(0, 300, 300)]
    sp = SampleParams(temperature=0.0, max_tokens=6)
    got = lm.generate(prompt, params=sp)
    assert got == lm.generate(prompt, 6)            # the greedy loop prefills too
    want, rec = oracle_generate_batch(P, embed, table, [prompt], [sp], seen_includes_prompt=True)
    assert_follows([got], want, rec, [sp])
    lm.close(); lm.backbone.close()


@pytest.mark.parametrize("plen", [5, 300])
def test_generate_streaming_hands_over_the_tokens_of_generate_one_by_one(plen):
    """generate == collecting generate_streaming's callback (gpu_lm.rs:323-331), for a stepped prompt and for one that
    takes the prefill route (where the first token exists before the first step); a callback may end the run early."""
    lm, P, embed, table = small_lm(1)
    rng = np.random.default_rng(plen)
    prompt = [int(t) for t in rng.integers(0, 300, plen)]
    sp = SampleParams(temperature=5.0, top_k=40, top_p=0.95, repetition_penalty=1.3, max_tokens=12, seed=21)
    want = lm.generate(prompt, params=sp)
    assert len(want) == 12
    got = []
    assert lm.generate_streaming(prompt, sp, got.append) is None
    assert got == want
    first = []
    lm.generate_streaming(prompt, sp, lambda t: first.append(t) or len(first) == 4)
    assert first == want[:4]
    # EOS ends the stream without being handed over (the reference breaks before the callback)
    eos = SampleParams(temperature=5.0, top_k=40, top_p=0.95, repetition_penalty=1.3, max_tokens=12, seed=21, eos_token_ids=[want[6]])
    cut = []
    lm.generate_streaming(prompt, eos, cut.append)
    assert cut == want[:want.index(want[6])]
    # an exception in the callback surfaces after the call, and the engine stays usable
    def boom(t):
        raise RuntimeError("stop")
    with pytest.raises(RuntimeError, match="stop"):
        lm.generate_streaming(prompt, sp, boom)
    assert lm.generate(prompt, params=sp) == want
    lm.close(); lm.backbone.close()


def test_generate_batch_rejects_bad_arguments():
    from mamba_rs_amd import MambaHipError
    lm, *_ = small_lm(2)
    with pytest.raises(ValueError):
        lm.generate_batch([[1]], [SampleParams()])
    with pytest.raises(MambaHipError, match="n_eos"):
        lm.generate_batch([[1], [2]], [SampleParams(eos_token_ids=list(range(17))), SampleParams()])
    lm.close(); lm.backbone.close()
