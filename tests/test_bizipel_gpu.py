"""Bizipel on the GPU against the plain implementation (tests/plain_bizipel.py): each mechanism's kernels alone, with
inputs made so that a wrong key, a window that is one token off, a lost state or a missing sink shows; then whole
models of three small configurations in 32-bit and in bfloat16: whole prompts, portions, token by token, unequal
batches, slots and pages used again, long decoding, the first tokens, and greedy generation through the pipeline."""
import math

import pytest
import torch

import plain_bizipel as P
from bizipel_cases import CONFIGS, model_folder, plain_logits, tokens_for
from helpers import assert_logits_close

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


def engine(name, dtype, max_tokens=1024, max_slots=None):
    from synaptix_amd import Engine
    return Engine.load(model_folder(name), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)


def dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


# ----------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("W", [72, 70])
@pytest.mark.parametrize("S", [1, 2, 5])
def test_streams_read_write_and_dynamic_tanh(S, W):
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(S)
    T = 37
    xs = torch.randn(S, T, W, generator=g, dtype=P.F64) * 3
    w_in, w_out = torch.randn(S, generator=g, dtype=P.F64), torch.randn(S, generator=g, dtype=P.F64)
    mix = torch.randn(S, S, generator=g, dtype=P.F64)
    alpha, gain, shift = torch.tensor(0.7, dtype=P.F64), torch.randn(W, generator=g, dtype=P.F64), torch.randn(W, generator=g, dtype=P.F64)
    X = dev(xs.permute(1, 0, 2))
    out = torch.empty((T, W), dtype=torch.float32, device=DEV)
    ops.streams_read_norm(X, dev(w_in), out, dyt=(dev(alpha.reshape(1)), dev(gain), dev(shift)))
    want = P.dynamic_tanh(P.streams_read(xs, w_in), alpha, gain, shift)
    assert float((out.cpu().double() - want).abs().max()) < 2e-5
    rows = torch.tensor([5, 0, 36], dtype=torch.int32, device=DEV)          # the sum of the streams on a few rows
    few = torch.empty((3, W), dtype=torch.float32, device=DEV)
    ops.streams_read_norm(X, None, few, rows=rows)
    assert float((few.cpu().double() - xs.sum(0)[[5, 0, 36]]).abs().max()) < 2e-5
    ya, yb = torch.randn(2, T, W, generator=g, dtype=P.F64), torch.randn(T, W, generator=g, dtype=P.F64)
    bias = torch.randn(W, generator=g, dtype=P.F64)
    ops.streams_update(X, dev(mix), dev(w_out), [(dev(ya), 0.8, dev(bias)), (dev(yb), -0.5, None)])
    want = P.streams_write(xs, mix, w_out, 0.8 * (ya.sum(0) + bias) - 0.5 * yb)
    assert float((X.cpu().double().permute(1, 0, 2) - want).abs().max()) < 5e-5
    # the same update with the next sublayer's read leaving in the same pass
    X2 = dev(xs.permute(1, 0, 2))
    nxt = torch.empty((T, W), dtype=torch.float32, device=DEV)
    w_next = torch.randn(S, generator=g, dtype=P.F64)
    ops.streams_update(X2, dev(mix), dev(w_out), [(dev(ya), 0.8, dev(bias)), (dev(yb), -0.5, None)],
                       read=(dev(w_next), (dev(alpha.reshape(1)), dev(gain), dev(shift)), nxt))
    assert torch.equal(X2, X)
    assert float((nxt.cpu().double() - P.dynamic_tanh(P.streams_read(want, w_next), alpha, gain, shift)).abs().max()) < 5e-5
    x0 = dev(xs[0])
    ops.streams_start(x0, X)
    assert torch.equal(X, x0.unsqueeze(1).expand(T, S, W))


def test_the_tanh_form_of_gelu_in_the_gated_feed_forward():
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    gu = torch.randn(9, 2 * 40, generator=g, dtype=P.F64) * 3
    out = torch.empty((9, 40), dtype=torch.float32, device=DEV)
    ops.swiglu(dev(gu), out, "gelu_tanh")
    assert float((out.cpu().double() - P.gelu_tanh(gu[:, :40]) * gu[:, 40:]).abs().max()) < 1e-5


def paged(k, v, dtype, shuffle_seed=0):
    """k [T, G, D], v [T, G, E] of one sequence -> (k_pages, v_pages, page_table [1, pages]) with the pages in a
    shuffled order and a page in front that belongs to nobody."""
    T, G, D = k.shape
    E = v.shape[2]
    n = -(-T // 64)
    order = torch.randperm(n, generator=torch.Generator().manual_seed(shuffle_seed)) + 1
    kp = torch.full((n + 1, G, 64, D), 50.0, dtype=torch.float32)          # what nobody may read is large
    vp = torch.full((n + 1, G, E, 64), 50.0, dtype=torch.float32)
    for t in range(T):
        kp[order[t // 64], :, t % 64, :] = k[t].float()
        vp[order[t // 64], :, :, t % 64] = v[t].float()
    return dev(kp, dtype), dev(vp, dtype), order.to(torch.int32).reshape(1, n).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep_first", [(96, 6), (64, 0), (65, 70), (7, 1), (0, 0)])
def test_window_attention_sees_exactly_its_keys(window, keep_first, dtype):
    """Keys are one-hot in one of four directions and queries point along their own key's direction with a large
    norm, so every query gives nearly all its weight to the visible keys of its own direction: a key that is
    wrongly seen or wrongly hidden at the window's edge, at the kept keys' edge or at a page's border changes the
    result by the order of the values themselves.  Prompt (all queries at once) and single tokens (the last queries alone)."""
    from synaptix_amd.kernels import ops
    T, H, G, D, E = 300, 4, 2, 8, 12
    g = torch.Generator().manual_seed(window * 7 + keep_first)
    kind = torch.randint(0, 4, (T,), generator=g)
    k = torch.zeros(T, G, D, dtype=P.F64)
    k[torch.arange(T), :, kind] = 1.0
    k += 0.01 * torch.randn(T, G, D, generator=g, dtype=P.F64)
    q = torch.zeros(T, H, D, dtype=P.F64)
    q[torch.arange(T), :, kind] = 6.0
    v = torch.randn(T, G, E, generator=g, dtype=P.F64)
    if dtype == torch.bfloat16:                     # the same rounded numbers for both sides
        q, k, v = (t.to(torch.bfloat16).double() for t in (q, k, v))
    r1, r2 = torch.tensor([0.3, 0.0, 1.0, 0.5], dtype=P.F64), torch.tensor([0.5, 2.0, 0.05, 1.0], dtype=P.F64)
    gate = torch.randn(T, H * E + 5, generator=g, dtype=P.F64)
    want = P.window_attention(q, k, v, 1.5, window or None, keep_first, r1, r2)
    want = want.reshape(T, H * E) * torch.sigmoid(gate[:, :H * E])
    kp, vp, table = paged(k, v, dtype)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    tok_pos = torch.arange(T, dtype=torch.int32, device=DEV)
    out = torch.empty((T, H * E), dtype=dtype, device=DEV)
    args = dict(window=window, keep_first=keep_first, sink_one=True, log_bias=(dev(r1), dev(r2)))
    ops.window_attention(dev(q.reshape(T, H * D), dtype), kp, vp, table, tok_seq, tok_pos, out, 1.5, H, G, D, E,
                         gate=dev(gate)[:, :H * E], **args)
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    assert float((out.cpu().double() - want).abs().max()) < tol
    last = 40                                       # the same queries one by one, as decoding sends them
    for t in range(T - last, T, 7):
        one = torch.empty((1, H * E), dtype=dtype, device=DEV)
        ops.window_attention(dev(q[t].reshape(1, H * D), dtype), kp, vp, table, tok_seq[:1], tok_pos[t:t + 1], one, 1.5,
                             H, G, D, E, gate=dev(gate)[t:t + 1, :H * E], **args)
        assert float((one.cpu().double() - want[t]).abs().max()) < tol
    # without the sink the weights sum to one: the plain softmax
    ops.window_attention(dev(q.reshape(T, H * D), dtype), kp, vp, table, tok_seq, tok_pos, out, 1.5, H, G, D, E,
                         window=window, keep_first=keep_first)
    plain = P.window_attention(q, k, v, 1.5, window or None, keep_first, sink_one=False).reshape(T, H * E)
    assert float((out.cpu().double() - plain).abs().max()) < tol


@pytest.mark.parametrize("D,E,window,keep_first", [(32, 16, 96, 6), (48, 48, 64, 0), (16, 80, 65, 70), (128, 128, 7, 1),
                                                   (64, 32, 0, 0)])
def test_window_attention_for_prompts_on_the_matrix_cores(D, E, window, keep_first):
    """The bf16 prompt kernel against the plain attention, with the peaked scores of the test above: three sequences of
    unequal lengths in one call, two of which continue from keys that an earlier portion left (the tiles begin inside
    a page, and their windows reach back into the old keys), and a sequence of one token."""
    from synaptix_amd.kernels import ops
    H, G = 4, 2
    g = torch.Generator().manual_seed(D + E + window)
    lens, pasts = [150, 1, 77, 203], [0, 0, 130, 61]
    r1, r2 = torch.tensor([0.3, 0.0, 1.0, 0.5], dtype=P.F64), torch.tensor([0.5, 2.0, 0.05, 1.0], dtype=P.F64)
    total = [n + p for n, p in zip(lens, pasts)]
    n_pages = [-(-t // 64) for t in total]
    kp = torch.full((sum(n_pages) + 1, G, 64, D), 50.0)
    vp = torch.full((sum(n_pages) + 1, G, E, 64), 50.0)
    table = torch.zeros((len(lens), max(n_pages)), dtype=torch.int32)
    order = (torch.randperm(sum(n_pages), generator=g) + 1).tolist()
    qs, wants, gates = [], [], []
    for b, T in enumerate(total):
        kind = torch.randint(0, 4, (T,), generator=g)
        k = 0.01 * torch.randn(T, G, D, generator=g, dtype=P.F64)
        k[torch.arange(T), :, kind] += 1.0
        q = torch.zeros(T, H, D, dtype=P.F64)
        q[torch.arange(T), :, kind] = 6.0
        v = torch.randn(T, G, E, generator=g, dtype=P.F64)
        q, k, v = (t.to(torch.bfloat16).double() for t in (q, k, v))
        gate = torch.randn(T, H * E, generator=g, dtype=P.F64)
        want = P.window_attention(q, k, v, 1.5, window or None, keep_first, r1, r2).reshape(T, H * E) * torch.sigmoid(gate)
        for pg in range(n_pages[b]):
            table[b, pg] = order.pop()
        for t in range(T):
            kp[table[b, t // 64], :, t % 64] = k[t].float()
            vp[table[b, t // 64], :, :, t % 64] = v[t].float()
        qs.append(q[pasts[b]:].reshape(lens[b], H * D))
        wants.append(want[pasts[b]:])
        gates.append(gate[pasts[b]:])
    start = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    out = torch.empty((sum(lens), H * E), dtype=torch.bfloat16, device=DEV)
    ops.window_attention_prefill_bf16(dev(torch.cat(qs), torch.bfloat16), dev(kp, torch.bfloat16), dev(vp, torch.bfloat16),
                                      table.to(DEV), start, torch.tensor(pasts, dtype=torch.int32, device=DEV), out, 1.5,
                                      H, G, D, E, window=window, keep_first=keep_first, sink_one=True,
                                      log_bias=(dev(r1), dev(r2)), gate=dev(torch.cat(gates)))
    err = (out.cpu().double() - torch.cat(wants)).abs()
    assert float(err.max()) < 1.5e-2, f"max err {float(err.max())} at row {int(err.max(1).values.argmax())}"


def test_window_intake_norms_q_and_k_and_writes_the_pages():
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    N, H, G, D, E = 70, 3, 1, 12, 20
    width = (H + G) * D + G * E + H * E
    proj, bias = torch.randn(N, width, generator=g, dtype=P.F64), torch.randn(width, generator=g, dtype=P.F64)
    qg, kg = torch.randn(D, generator=g, dtype=P.F64), torch.randn(D, generator=g, dtype=P.F64)
    x = proj + bias
    q = P.unit_rms(x[:, :H * D].view(N, H, D), 1e-5) * qg
    k = P.unit_rms(x[:, H * D:(H + G) * D].view(N, G, D), 1e-5) * kg
    v = x[:, (H + G) * D:(H + G) * D + G * E].view(N, G, E)
    # two sequences: tokens 0..29 at positions 50..79 of sequence 1 (over a page's border), the rest at 0.. of sequence 0
    tok_seq = torch.tensor([1] * 30 + [0] * 40, dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor(list(range(50, 80)) + list(range(40)), dtype=torch.int32, device=DEV)
    table = torch.tensor([[3, 0], [1, 2]], dtype=torch.int32, device=DEV)
    kp = torch.zeros((4, G, 64, D), dtype=torch.float32, device=DEV)
    vp = torch.zeros((4, G, E, 64), dtype=torch.float32, device=DEV)
    q_out = torch.empty((N, H * D), dtype=torch.float32, device=DEV)
    ops.window_intake(dev(proj), dev(bias), q_out, kp, vp, table, tok_seq, tok_pos, dev(qg), dev(kg), 1e-5, H, G, D, E)
    assert float((q_out.cpu().double() - q.reshape(N, H * D)).abs().max()) < 1e-5
    kp, vp = kp.cpu().double(), vp.cpu().double()
    for n in range(N):
        seq, pos = int(tok_seq[n]), int(tok_pos[n])
        page = int(table[seq, pos // 64])
        assert float((kp[page, :, pos % 64] - k[n]).abs().max()) < 1e-5
        assert float((vp[page, :, :, pos % 64] - v[n]).abs().max()) < 1e-5


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("H,D,E,T", [(2, 10, 72, 150), (1, 64, 16, 40), (3, 5, 130, 33), (1, 130, 64, 70)])
def test_matrix_memory_in_portions_and_slots(H, D, E, T, chunked):
    """Two sequences in one step (their states in rows 2 and 0), then the rest of both in a second step from the
    states the first left; gates drawn wide so that the running maximum moves and old contents decay."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 100 + D)
    cap, width = 6.0, 2 * H * D + 2 * H * E + 2 * H
    size = ops.matrix_memory_state_size(D, E)
    state = torch.zeros((4, H, size), dtype=torch.float32, device=DEV)
    state[1] = 7.0                                           # a row that belongs to nobody stays as it is
    seqs = {}
    for s, n in ((2, T), (0, T // 3)):
        proj = torch.randn(n, width, generator=g, dtype=P.F64)
        proj[:, -2 * H:] *= 8.0
        ib, fb = torch.randn(H, generator=g, dtype=P.F64), torch.randn(H, generator=g, dtype=P.F64) + 2.0
        seqs[s] = (proj, ib, fb)
    ib, fb = seqs[2][1], seqs[2][2]

    def plain(proj):
        n = proj.shape[0]
        q = proj[:, :H * D].view(n, H, D) * D ** -0.5
        k = proj[:, H * D:2 * H * D].view(n, H, D)
        v = proj[:, 2 * H * D:2 * H * D + H * E].view(n, H, E)
        return P.matrix_memory(q, k, v, proj[:, -2 * H:-H] + ib, proj[:, -H:] + fb, cap)

    want = {s: plain(seqs[s][0]) for s in seqs}
    cut = {2: T // 2 + 1, 0: 2}
    got = {s: [] for s in seqs}
    for part in (0, 1):
        pieces = [seqs[s][0][:cut[s]] if part == 0 else seqs[s][0][cut[s]:] for s in (2, 0)]
        proj = dev(torch.cat(pieces))
        start = torch.tensor([0, pieces[0].shape[0], proj.shape[0]], dtype=torch.int32, device=DEV)
        slot = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
        out = torch.empty((proj.shape[0], H * E), dtype=torch.float32, device=DEV)
        ops.matrix_memory_scan(proj, dev(ib), dev(fb), cap, D ** -0.5, state, start, slot, out, H, D, E, chunked=chunked)
        got[2].append(out[:pieces[0].shape[0]])
        got[0].append(out[pieces[0].shape[0]:])
    for s in seqs:
        o = torch.cat(got[s]).cpu().double().view(-1, H, E)
        # (o is a quotient whose divisor n . q cancels now and then: where it does, a last-bit difference in a sum
        # is a larger one in o, so the bound on o is wider than the one on the state below)
        scale = float(want[s][0].abs().max())
        assert float((o - want[s][0]).abs().max()) < 6e-5 * max(1.0, scale)
        C, n, m = want[s][1]
        st = state[s].cpu().double()
        assert float((st[:, :D * E].view(H, D, E) - C).abs().max()) < 2e-5 * max(1.0, float(C.abs().max()))
        assert float((st[:, D * E:D * E + D] - n).abs().max()) < 2e-5 * max(1.0, float(n.abs().max()))
        assert float((st[:, -1] - m).abs().max()) < 1e-5
    assert float((state[1] - 7.0).abs().max()) == 0.0
    # the heads' unit norm, gain and gate
    o = want[2][0]
    gain, gate = torch.randn(H * E, generator=g, dtype=P.F64), torch.randn(T, H * E + 3, generator=g, dtype=P.F64)
    out = torch.empty((T, H * E), dtype=torch.float32, device=DEV)
    ops.head_norm_gate(dev(o.reshape(T, H * E)), dev(gain), 1e-6, dev(gate)[:, :H * E], out, H, E)
    ref = P.unit_rms(o, 1e-6).reshape(T, H * E) * gain * torch.sigmoid(gate[:, :H * E])
    assert float((out.cpu().double() - ref).abs().max()) < 2e-5


# ----------------------------------------------------------------------------- whole models

def lengths(name):
    return {"P": [1, 2, 21, 64, 65, 150], "Q": [3, 70, 71, 129, 140], "R": [5, 64, 128, 200], "S": [1, 12, 66, 90],
            "T": [2, 31, 64, 100], "U": [1, 7, 65, 80]}[name]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "T", "U"])
def test_whole_prompts(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        toks = tokens_for(name, n, 100 + i)
        s = eng.acquire()
        got = eng.step([(s, toks)], want="all")
        assert_logits_close(got, plain_logits(name, toks), dtype, f"{name} {dtype} {n} tokens whole", sharp=True)
        eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_portions_of_several_sizes(name, dtype):
    """A prompt in portions of 2, 1, 3, 17, 64 and 2 tokens and the rest: every portion starts from the cache and the
    state that the earlier ones left (inside a page, at a page's border, inside and beyond the first window)."""
    toks = tokens_for(name, 230, 7)
    want = plain_logits(name, toks)
    eng = engine(name, dtype)
    s, at, got = eng.acquire(), 0, []
    for n in [2, 1, 3, 17, 64, 2, 41, 100]:
        got.append(eng.step([(s, toks[at:at + n])], want="all"))
        at += n
    assert at == len(toks)
    assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} in portions", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,head,n", [("P", 30, 130), ("Q", 1, 160), ("R", 100, 140), ("S", 3, 90), ("T", 40, 110)])
def test_prompt_then_token_by_token(name, head, n, dtype):
    """Decoding long enough that every window passes over decoded tokens and over a page's border, that the kept first
    keys are the only old ones left, and that the state has been carried over a hundred steps."""
    toks = tokens_for(name, n, 21)
    want = plain_logits(name, toks)
    eng = engine(name, dtype)
    s = eng.acquire()
    got = [eng.step([(s, toks[:head])], want="all")]
    for t in toks[head:]:
        got.append(eng.step([(s, [t])], want="last"))
    assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} token by token", sharp=True)
    eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "T", "U"])
def test_unequal_batches_and_slots_used_again(name, dtype):
    """Requests of unequal lengths start together and are decoded together, the shorter ones ending earlier; then
    other requests take the slots and pages that came free (the cache has room for little more than one batch), in
    another order: each request's logits equal the plain model's for that request alone."""
    reqs = {f"r{i}": tokens_for(name, n + 9, 300 + i) for i, n in enumerate(lengths(name))}
    ids = list(reqs)
    eng = engine(name, dtype, max_tokens=64 * 9, max_slots=3)
    for batch in (ids[:3], (ids[3:] + ids[:1])[:3], list(reversed(ids))[:3]):
        slots = {r: eng.acquire() for r in batch}
        head = {r: max(1, len(reqs[r]) - 9 - 3 * i) for i, r in enumerate(batch)}
        got = {r: [] for r in batch}
        out = eng.step([(slots[r], reqs[r][:head[r]]) for r in batch], want="all")
        at = 0
        for r in batch:
            got[r].append(out[at:at + head[r]])
            at += head[r]
        fed, live = dict(head), list(batch)
        while live:
            out = eng.step([(slots[r], [reqs[r][fed[r]]]) for r in live], want="last")
            for i, r in enumerate(live):
                got[r].append(out[i:i + 1])
                fed[r] += 1
            for r in [r for r in live if fed[r] == len(reqs[r])]:
                eng.release(slots[r])
                live.remove(r)
        for r in batch:
            assert_logits_close(torch.cat(got[r]), plain_logits(name, reqs[r]), dtype, f"{name} {dtype} {r} in a batch",
                                sharp=True)
        eng.cache.check()
    assert eng.cache.free_slots == 3


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens(dtype):
    """Sequences of one and two tokens, and every position up to the kept keys, the window and a little more."""
    for name in ("P", "Q"):
        eng = engine(name, dtype)
        toks = tokens_for(name, 30, 77)
        want = plain_logits(name, toks)
        for n in (1, 2):
            s = eng.acquire()
            assert_logits_close(eng.step([(s, toks[:n])], want="all"), plain_logits(name, toks[:n]), dtype,
                                f"{name} {dtype} first {n}", sharp=True)
            eng.release(s)
        s = eng.acquire()
        got = [eng.step([(s, [t])], want="last") for t in toks]
        assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} from the first token one by one", sharp=True)


def test_long_decoding_in_float32():
    toks = tokens_for("P", 700, 5)
    want = plain_logits("P", toks)
    eng = engine("P", "float32", max_tokens=64 * 4)      # the windows give their pages back: four pages are enough
    s = eng.acquire()
    got = [eng.step([(s, toks[:2])], want="all")]
    for t in toks[2:]:
        got.append(eng.step([(s, [t])], want="last"))
    assert_logits_close(torch.cat(got), want, "float32", "700 tokens one by one", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_pipeline(dtype):
    """Pipeline.generate_batch (the scheduler, slots, eager decode steps, the sampler) against greedy decoding with the
    plain model; in bfloat16 a token may differ where the two best logits are close, then the plain model's logits
    for the generated sequence must say so."""
    import synaptix_amd
    name = "R"
    pipe = synaptix_amd.load(model_folder(name), dtype="f32" if dtype == "float32" else "bf16", max_seq=512)
    prompts = [tokens_for(name, n, 900 + n) for n in (3, 70, 20)]
    outs, stats = pipe.generate_batch(prompts, synaptix_amd.GenerationConfig(max_new_tokens=12, temperature=0.0))
    assert stats.new_tokens == 36
    for prompt, out in zip(prompts, outs):
        assert len(out.tokens) == 12 and out.finish_reason == "length"
        logits = plain_logits(name, prompt + out.tokens)
        for i, tok in enumerate(out.tokens):
            row = logits[len(prompt) - 1 + i]
            best = int(row.argmax())
            if dtype == "float32":
                assert tok == best or float(row[best] - row[tok]) < 1e-4
            else:
                assert tok == best or float(row[best] - row[tok]) < 0.05 * float(row.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "R"])
def test_decode_steps_replayed_from_a_graph(name, dtype):
    """Captured decode steps (three rows wide in a graph of four: one row is padding) with eager work of other
    sequences between the replays; every replay against the plain model, and the states of the sequences that a
    capture ran twice must be where a single step leaves them."""
    eng = engine(name, dtype, max_tokens=64 * 12)
    assert eng.graph_ok
    reqs = [tokens_for(name, n, 40 + n) for n in (90, 20, 140)]
    other = tokens_for(name, 60, 4)
    want = [plain_logits(name, r) for r in reqs]
    heads = [len(r) - 12 for r in reqs]
    slots = [eng.acquire() for _ in reqs]
    eng.step([(s, r[:h]) for s, r, h in zip(slots, reqs, heads)], want=None)
    runner = eng.decode_runner(3, 256)
    assert runner.rows == 4
    extra = eng.acquire()
    for i in range(12):
        _, lg = runner.step(slots, [r[h + i] for r, h in zip(reqs, heads)])
        for j in range(3):
            assert_logits_close(lg[j:j + 1].clone(), want[j][heads[j] + i:heads[j] + i + 1], dtype,
                                f"{name} {dtype} replay {i} row {j}", sharp=True)
        got = eng.step([(extra, other[5 * i:5 * i + 5])], want="last")        # an eager prompt portion in between
        assert_logits_close(got, plain_logits(name, other)[5 * i + 4:5 * i + 5], dtype, f"{name} {dtype} eager between replays",
                            sharp=True)
    eng.cache.check()


def test_short_prompt_steps_replayed_from_a_graph():
    """bfloat16 prompt steps of a few tokens go through captured graphs with padding rows (an extra sequence on the
    spare page and the spare state row); portions of a prompt one after another, each from what the last one left."""
    name = "R"
    eng = engine(name, "bfloat16")
    assert eng.graph_ok and eng.prompt_graphs
    toks = tokens_for(name, 120, 8)
    want = plain_logits(name, toks)
    s, at = eng.acquire(), 0
    for n in (10, 10, 30, 10, 40, 20):
        got = eng.step([(s, toks[at:at + n])], want="last")
        at += n
        assert_logits_close(got, want[at - 1:at], "bfloat16", f"prompt portion ending at {at} through a graph", sharp=True)
    assert any(k[0] == "prompt" for k in eng._runners), "no prompt step was replayed from a graph"


def test_command_line_and_trace_replay_as_a_user_starts_them(tmp_path):
    """`random` writes a model folder from a configuration file, `run` generates from it, and bin/trace_run replays
    steps over it (prompts of unequal lengths together, then single tokens, a request that ends early, its slot used
    again by a later request) in both types; the logits against the plain model, the generated tokens against its
    greedy choice."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from helpers import ROOT, batched_trace
    from plain_bizipel import PlainBizipel

    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(CONFIGS["P"]))
    folder = str(tmp_path / "model")
    env = dict(os.environ, PYTHONPATH=ROOT)
    subprocess.run([sys.executable, "-m", "synaptix_amd", "random", str(cfg_file), folder, "--seed", "3"], check=True,
                   env=env, cwd=ROOT, timeout=300)
    plain = PlainBizipel.from_folder(folder)
    prompt = tokens_for("P", 9, 1)
    run = subprocess.run([sys.executable, "-m", "synaptix_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)),
                          "--max-tokens", "6", "--temperature", "0", "--compute-dtype", "f32"], check=True, env=env,
                         cwd=ROOT, timeout=300, capture_output=True, text=True)
    out = [int(t) for t in run.stdout.split()]
    assert len(out) == 6
    logits = plain.forward(prompt + out)
    for i, tok in enumerate(out):
        row = logits[len(prompt) - 1 + i]
        assert tok == int(row.argmax()) or float(row.max() - row[tok]) < 1e-4

    reqs = {"a": tokens_for("P", 75, 2), "b": tokens_for("P", 8, 3), "c": tokens_for("P", 130, 4), "d": tokens_for("P", 40, 5)}
    steps, where = batched_trace(reqs, [["a", "b", "c"], ["d", "b"]], decode=5)
    for dtype in DTYPES:
        out_dir = str(tmp_path / dtype)
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                               "--out", out_dir, "--max-tokens", "640"], input="".join(json.dumps(s) + "\n" for s in steps),
                              capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
        got = {s["step"]: np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4").reshape(-1, CONFIGS["P"]["vocab"])
               for s in steps}
        for rid, toks in reqs.items():
            want = plain.forward(toks)
            rows = np.stack([got[where[(rid, p)][0]][where[(rid, p)][1]] for p in range(len(toks))])
            assert_logits_close(rows, want, dtype, f"trace_run {dtype} request {rid}", sharp=False)
