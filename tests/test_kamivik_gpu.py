"""Kamivik on the GPU against the plain implementation (tests/plain_kamivik.py): each mechanism's kernels alone, with
inputs made so that a wrong key, a window that is one token off or a wrong expert shows; then whole models of five
small configurations in 32-bit and in bfloat16: whole prompts, portions, token by token, unequal batches, slots and
pages used again, long decoding, the first tokens, and greedy generation through the pipeline."""
import math

import pytest
import torch

import plain_kamivik as P
from kamivik_cases import CONFIGS, cases, model_folder, plain_logits, plain_model, tokens_for
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


def rounded(dtype, *ts):
    """The same numbers for both sides: what the type can hold."""
    return [t.to(dtype).double() for t in ts]


# ----------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("W", [64, 70])
def test_scaled_terms_into_the_residual_and_the_norm(W):
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(W)
    T = 19
    x = torch.randn(T, W, generator=g, dtype=P.F64)
    a, b = torch.randn(3, T, W, generator=g, dtype=P.F64), torch.randn(T, W, generator=g, dtype=P.F64)
    s1, s2 = torch.randn(W, generator=g, dtype=P.F64), torch.randn(W, generator=g, dtype=P.F64)
    gain = torch.randn(W, generator=g, dtype=P.F64)
    want_x = x + s1 * a.sum(0) + s2 * b
    want = P.rms_norm(want_x, gain, 1e-5)
    X, out = dev(x), torch.empty((T, W), dtype=torch.float32, device=DEV)
    ops.add_scaled_rmsnorm(X, [(dev(a), dev(s1)), (dev(b), dev(s2))], dev(gain), 1e-5, out)
    assert float((X.cpu().double() - want_x).abs().max()) < 1e-5 and float((out.cpu().double() - want).abs().max()) < 1e-5
    # a few rows only: the residual stays; one term without a scale; no norm at all
    X = dev(x)
    rows = torch.tensor([4, 0, 18], dtype=torch.int32, device=DEV)
    few = torch.empty((3, W), dtype=torch.bfloat16, device=DEV)
    ops.add_scaled_rmsnorm(X, [(dev(b), None)], dev(gain), 1e-5, few, rows=rows)
    assert torch.equal(X, dev(x))
    assert float((few.cpu().double() - P.rms_norm(x + b, gain, 1e-5)[[4, 0, 18]]).abs().max()) < 3e-2
    ops.add_scaled_rmsnorm(X, [(dev(a), dev(s1))], None, 0.0, None)
    assert float((X.cpu().double() - (x + s1 * a.sum(0))).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,H,K,J", [(70, 3, 32, 40), (5, 2, 64, 16), (33, 4, 20, 7), (1, 1, 96, 130), (130, 2, 128, 64),
                                     (100, 2, 40, 24), (300, 1, 72, 200)])
def test_a_linear_map_for_each_head(N, H, K, J, dtype):
    """In bf16 on the matrix cores: tiles through LDS from 48 rows on (any K that is a multiple of 8, a last k-tile
    that is partly empty), operands straight from memory for fewer rows (K a multiple of 32); plain FMA otherwise;
    into a piece of longer rows; with one gate a head and with one gate a value."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(N + K)
    x, w = rounded(dtype, torch.randn(N, H, K, generator=g), torch.randn(H, J, K, generator=g) / math.sqrt(K))
    gate = torch.randn(N, 3 + H * J, generator=g, dtype=P.F64)
    plain = torch.einsum("nhk,hjk->nhj", x, w)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    out = torch.full((N, H, J + 5), 7.0, dtype=dtype, device=DEV)
    ops.heads_product(dev(x, dtype), dev(w, dtype), out, out_offset=3)
    assert float((out[:, :, 3:3 + J].cpu().double() - plain).abs().max()) < tol
    assert bool((out[:, :, :3] == 7).all()) and bool((out[:, :, 3 + J:] == 7).all())
    G = dev(gate)
    out = torch.empty((N, H, J), dtype=dtype, device=DEV)
    ops.heads_product(dev(x, dtype), dev(w, dtype), out, gate=G[:, 3:], gate_per_value=True)
    assert float((out.cpu().double() - plain * torch.sigmoid(gate[:, 3:]).view(N, H, J)).abs().max()) < tol
    ops.heads_product(dev(x, dtype), dev(w, dtype), out, gate=G[:, 1:1 + H], gate_per_value=False)
    assert float((out.cpu().double() - plain * torch.sigmoid(gate[:, 1:1 + H])[:, :, None]).abs().max()) < tol
    if dtype == torch.bfloat16:           # all kernels give the sums of the same products
        for force in (1, 2, 3):           # plain FMA; the matrix cores without LDS (where K allows, else FMA again)
            other = torch.empty_like(out)
            ops.heads_product(dev(x, dtype), dev(w, dtype), other, gate=G[:, 1:1 + H], gate_per_value=False, force_simt=force)
            assert float((other.float() - out.float()).abs().max()) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,W,F,E,top", [(50, 64, 32, 6, 2), (3, 40, 24, 5, 5), (1, 32, 96, 4, 1), (200, 96, 64, 16, 3),
                                         (9, 72, 20, 1, 1), (300, 64, 40, 4, 2)])
def test_router_and_experts(N, W, F, E, top, dtype):
    """The router's logits are spread so that no choice is close; an expert that nobody chose has an empty segment."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(N * E)
    h, wr = rounded(dtype, torch.randn(N, W, generator=g), torch.randn(E, W, generator=g))
    bias = 3.0 * torch.randn(E, generator=g, dtype=P.F64)
    if E > 3:
        bias[2] = -1e4                                  # nobody's choice
    ups, downs = rounded(dtype, torch.randn(E, F, W, generator=g) / math.sqrt(W), torch.randn(E, W, F, generator=g) / math.sqrt(F))
    want_ids, want_w = P.route(h, wr, bias, top)
    ids = torch.empty((N, top), dtype=torch.int32, device=DEV)
    weights = torch.empty((N, top), dtype=torch.float32, device=DEV)
    from synaptix_amd.parts import linear, Matrix
    ops.route_topk(linear(dev(h, dtype), Matrix(dev(wr, dtype)), torch.float32), dev(bias), ids, weights)
    assert torch.equal(ids.cpu().long(), want_ids)
    assert float((weights.cpu().double() - want_w).abs().max()) < 1e-4
    seg, tok_of, pair_of, part_of, weight_of = ops.route_sort(ids, weights, E)
    seg_h, tok_h, pair_h = seg.cpu().tolist(), tok_of.cpu().tolist(), pair_of.cpu().tolist()
    assert seg_h[0] == 0 and seg_h[-1] == N * top and sorted(pair_h) == list(range(N * top))
    for e in range(E):
        for r in range(seg_h[e], seg_h[e + 1]):
            assert int(want_ids.view(-1)[pair_h[r]]) == e and tok_h[r] == pair_h[r] // top
    assert part_of.cpu().tolist() == [(p % top) * N + p // top for p in pair_h]
    assert torch.equal(weight_of.cpu(), weights.view(-1).cpu()[pair_of.cpu().long()])
    want = torch.zeros(N, W, dtype=P.F64)
    for t in range(N):
        for e, a in zip(want_ids[t].tolist(), want_w[t]):
            want[t] += a * (downs[e] @ P.gelu(ups[e] @ h[t]))
    w_up, w_down = dev(ups, dtype), dev(downs, dtype)
    kept = [(w_up, w_down)]
    if dtype == torch.bfloat16 and ops.pack_expert_weights(w_up) is not None and ops.pack_expert_weights(w_down) is not None:
        kept.append((ops.pack_expert_weights(w_up), ops.pack_expert_weights(w_down)))      # in fragment order
    for w_up, w_down in kept:
        for force in (0, 1, 2, 3):      # by size; plain FMA; the matrix cores without LDS, 16 and 64 outputs a wave
            mid = torch.empty((N * top, F), dtype=dtype, device=DEV)
            ops.experts_product(dev(h, dtype), w_up, mid, seg, tok_of, pair_of, gelu=True, force_simt=force)
            y = torch.empty((top, N, W), dtype=torch.float32, device=DEV)
            ops.experts_product(mid, w_down, y.view(top * N, W), seg, pair_of, part_of, row_weight=weight_of,
                                force_simt=force)
            assert float((y.sum(0).cpu().double() - want).abs().max()) < (5e-5 if dtype == torch.float32 else 5e-2)


def paged_rows(rows, n_values, dtype, shuffle_seed=0):
    """rows [T, R] of one sequence -> (k_pages [pages, 1, 64, R], v_pages [pages, 1, n_values, 64], page_table [1,
    pages]) with the pages in a shuffled order and a page in front that belongs to nobody."""
    T, R = rows.shape
    n = -(-T // 64)
    order = torch.randperm(n, generator=torch.Generator().manual_seed(shuffle_seed)) + 1
    kp = torch.full((n + 1, 1, 64, R), 50.0, dtype=torch.float32)          # what nobody may read is large
    vp = torch.full((n + 1, 1, n_values, 64), 50.0, dtype=torch.float32)
    for t in range(T):
        kp[order[t // 64], 0, t % 64, :] = rows[t].float()
        vp[order[t // 64], 0, :, t % 64] = rows[t, :n_values].float()
    return dev(kp, dtype), dev(vp, dtype), order.to(torch.int32).reshape(1, n).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 1, 2, 63, 64, 65, 130, 1000])
def test_latent_attention_sees_exactly_its_keys(window, dtype):
    """Key rows point in one of four directions and queries along their own row's direction with a large norm, so every
    query gives nearly all its weight to the visible rows of its own direction: a row wrongly seen or wrongly hidden
    at the window's edge or at a page's border changes the result by the order of the values themselves.  One
    direction has a single row, far back at position 2: queries along it, hundreds of rows later, find it among all
    the others or, with a window, must not.  All queries at once, and the last ones alone as decoding sends them."""
    from synaptix_amd.kernels import ops
    T, H, C, B = 300, 3, 12, 4
    R = C + B
    g = torch.Generator().manual_seed(window + 1)
    kind = torch.randint(0, 3, (T,), generator=g)
    kind[2] = 3
    rows = 0.05 * torch.randn(T, R, generator=g, dtype=P.F64)
    rows[torch.arange(T), C - 2 + kind] += 1.0                   # directions C-2 .. C+1: two in the latent, two behind it
    rows[:, :C - 2] += torch.randn(T, C - 2, generator=g, dtype=P.F64)    # what the values carry
    q = torch.zeros(T, H, R, dtype=P.F64)
    q[torch.arange(T), :, C - 2 + kind] = 8.0
    far = [150, 299, 64, 66]
    for t in far:
        q[t] = 0
        q[t, :, C + 1] = 12.0                                    # along the single row at position 2
    q, rows = rounded(dtype, q, rows)
    want = P.shared_row_attention(q, rows, C, 1.25, window or None)
    kp, vp, table = paged_rows(rows, C, dtype, shuffle_seed=window)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    tok_pos = torch.arange(T, dtype=torch.int32, device=DEV)
    out = torch.empty((T, H * C), dtype=dtype, device=DEV)
    ops.latent_attention(dev(q.reshape(T, H * R), dtype), kp, vp, table, tok_seq, tok_pos, out, 1.25, H, C, B, window=window)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert float((out.cpu().double().view(T, H, C) - want).abs().max()) < tol
    if window == 0:               # the far row is what those queries return
        assert float((want[299, 0] - rows[2, :C]).abs().max()) < 1e-2
    for t in sorted(set(far + list(range(T - 40, T, 7)) + [0, 1, 63, 64, 65])):
        one = torch.empty((1, H * C), dtype=dtype, device=DEV)
        ops.latent_attention(dev(q[t].reshape(1, H * R), dtype), kp, vp, table, tok_seq[:1], tok_pos[t:t + 1], one, 1.25,
                             H, C, B, window=window)
        assert float((one.cpu().double().view(H, C) - want[t]).abs().max()) < tol, f"query {t} alone"


def test_latent_attention_over_long_rows_in_float32():
    """Rows of 320 + 40 values through the plain kernel (its instantiation for head sizes above 256): random rows, the
    queries long enough that the softmax is peaked; all queries at once and one alone."""
    from synaptix_amd.kernels import ops
    T, H, C, B, window = 150, 2, 320, 40, 65
    g = torch.Generator().manual_seed(9)
    rows = torch.randn(T, C + B, generator=g, dtype=P.F64)
    q = torch.randn(T, H, C + B, generator=g, dtype=P.F64) * 0.5
    want = P.shared_row_attention(q, rows, C, 0.3, window)
    kp, vp, table = paged_rows(rows, C, torch.float32, shuffle_seed=3)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    tok_pos = torch.arange(T, dtype=torch.int32, device=DEV)
    out = torch.empty((T, H * C), dtype=torch.float32, device=DEV)
    ops.latent_attention(dev(q.reshape(T, -1)), kp, vp, table, tok_seq, tok_pos, out, 0.3, H, C, B, window=window)
    assert float((out.cpu().double().view(T, H, C) - want).abs().max()) < 5e-5
    one = torch.empty((1, H * C), dtype=torch.float32, device=DEV)
    ops.latent_attention(dev(q[140].reshape(1, -1)), kp, vp, table, tok_seq[:1], tok_pos[140:141], one, 0.3, H, C, B, window=window)
    assert float((one.cpu().double().view(H, C) - want[140]).abs().max()) < 5e-5


@pytest.mark.parametrize("H,C,B", [(3, 16, 16), (16, 32, 16), (5, 48, 0), (2, 144, 48), (20, 256, 64), (4, 512, 64)])
@pytest.mark.parametrize("window", [0, 1, 64, 65, 130])
def test_latent_attention_in_tiles_on_the_matrix_cores(window, H, C, B):
    """The bf16 kernel whose tiles are 16 (token, head) rows of one sequence, for every size of its register tiles, with
    k-steps of 16 and of 32: two sequences in one step, the second (470 rows) continuing from 70 cached rows (a portion that
    starts inside a page); then single tokens of both sequences together, whose pages are cut into splits and merged.
    Rows and queries as in the test above (a wrong or lost key shows); slots behind a sequence's end hold NaN."""
    from synaptix_amd.kernels import ops
    R, dt = C + B, torch.bfloat16
    lens, past = [150, 470], [0, 70]
    g = torch.Generator().manual_seed(window + H)
    qs, rowss, wants = [], [], []
    for T in lens:
        kind = torch.randint(0, 3, (T,), generator=g)
        kind[2] = 3
        rows = 0.05 * torch.randn(T, R, generator=g, dtype=P.F64)
        rows[torch.arange(T), C - 4 + kind] += 1.0
        rows[:, :C - 4] += torch.randn(T, C - 4, generator=g, dtype=P.F64)
        q = torch.zeros(T, H, R, dtype=P.F64)
        q[torch.arange(T), :, C - 4 + kind] = 8.0
        for t in (T - 1, T - 30, 100):
            q[t] = 0
            q[t, :, C - 1] = 12.0
        q, rows = rounded(dt, q, rows)
        qs.append(q), rowss.append(rows), wants.append(P.shared_row_attention(q, rows, C, 1.25, window or None))
    # the two sequences' pages side by side in one pool; what lies behind a sequence's end is NaN
    pools = [paged_rows(r, C, torch.float32, shuffle_seed=5 + j) for j, r in enumerate(rowss)]
    n0 = pools[0][0].shape[0]
    kp = torch.cat([pools[0][0], pools[1][0]]).float()
    vp = torch.cat([pools[0][1], pools[1][1]]).float()
    width = max(p[2].shape[1] for p in pools)
    table = torch.zeros((2, width), dtype=torch.int32, device=DEV)
    for j, (_, _, tb) in enumerate(pools):
        table[j, :tb.shape[1]] = tb[0] + (n0 if j else 0)
        last, used = int(table[j, (lens[j] - 1) // 64]), (lens[j] - 1) % 64 + 1
        kp[last, 0, used:] = float("nan")
        vp[last, 0, :, used:] = float("nan")
    kp, vp = kp.to(dt), ops.latent_v_pages_to_kernel_order(vp.to(dt))
    new = [lens[0] - past[0], lens[1] - past[1]]
    q_step = torch.cat([qs[0][past[0]:], qs[1][past[1]:]]).reshape(-1, H * R)
    want = torch.cat([wants[0][past[0]:], wants[1][past[1]:]])
    seqs = (torch.tensor([0, new[0], new[0] + new[1]], dtype=torch.int32, device=DEV),
            torch.tensor(past, dtype=torch.int32, device=DEV))
    out = torch.empty((q_step.shape[0], H * C), dtype=dt, device=DEV)
    ops.latent_attention(dev(q_step, dt), kp, vp, table, None, None, out, 1.25, H, C, B, window=window, seqs=seqs)
    assert float((out.cpu().double().view(-1, H, C) - want).abs().max()) < 2e-2
    # the last tokens alone, one of each sequence: their pages in splits
    for back in (1, 30):
        q1 = torch.stack([qs[0][lens[0] - back], qs[1][lens[1] - back]]).reshape(2, H * R)
        seqs1 = (torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV),
                 torch.tensor([lens[0] - back, lens[1] - back], dtype=torch.int32, device=DEV))
        assert ops.latent_attention_workspace(2, H, 2, C, width) > 0
        one = torch.empty((2, H * C), dtype=dt, device=DEV)
        ops.latent_attention(dev(q1, dt), kp, vp, table, None, None, one, 1.25, H, C, B, window=window, seqs=seqs1)
        w1 = torch.stack([wants[0][lens[0] - back], wants[1][lens[1] - back]])
        assert float((one.cpu().double().view(2, H, C) - w1).abs().max()) < 2e-2, f"single tokens {back} from the end"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,B,C,pairs", [(3, 8, 6, 20, 3), (2, 16, 8, 32, 2), (1, 4, 0, 6, 0), (4, 32, 16, 64, 8)])
def test_latent_intake_norms_turns_and_writes_the_pages(H, D, B, C, pairs, dtype):
    from synaptix_amd.kernels import ops
    from synaptix_amd.parts import RotaryInterleaved
    g = torch.Generator().manual_seed(H * C)
    N, R = 7, C + B
    width = H * (D + B) + R + 5
    proj = torch.randn(N, width, generator=g, dtype=P.F64)
    gain = torch.randn(C, generator=g, dtype=P.F64)
    seqs, pos = [0, 0, 1, 0, 1, 1, 1], [63, 64, 0, 65, 1, 2, 3]       # two sequences, one over a page's border
    table = torch.tensor([[2, 1], [3, 0]], dtype=torch.int32, device=DEV)
    kp = torch.zeros((4, 1, 64, R), dtype=dtype, device=DEV)
    vp = torch.zeros((4, 1, C, 64), dtype=dtype, device=DEV)
    qn = torch.empty((N, H * D), dtype=dtype, device=DEV)
    qf = torch.full((N, H * R), 9.0, dtype=dtype, device=DEV)
    cos, sin = RotaryInterleaved(70.0, 2 * pairs, 128).tables(DEV) if pairs else (None, None)
    ops.latent_intake(dev(proj), dev(gain), 1e-5, cos, sin, qn, qf, kp, vp, table,
                      torch.tensor(seqs, dtype=torch.int32, device=DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
                      H, D, B, C, max(pos))
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    P_t = torch.tensor(pos)
    q = proj[:, :H * (D + B)].view(N, H, D + B)
    assert float((qn.cpu().double().view(N, H, D) - q[..., :D]).abs().max()) < tol
    if B:
        assert float((qf.cpu().double().view(N, H, R)[..., C:] - P.turn_pairs(q[..., D:], P_t, 70.0, 2 * pairs)).abs().max()) < tol
    assert bool((qf.view(N, H, R)[..., :C] == 9).all())                 # the absorbed query's places are left alone
    down = proj[:, H * (D + B):H * (D + B) + R]
    want_row = torch.cat([P.rms_norm(down[:, :C], gain, 1e-5), P.turn_pairs(down[:, C:], P_t, 70.0, 2 * pairs)], -1)
    pages = table.cpu()
    for n in range(N):
        page, slot = int(pages[seqs[n], pos[n] // 64]), pos[n] % 64
        assert float((kp[page, 0, slot].cpu().double() - want_row[n]).abs().max()) < tol
        assert float((vp[page, 0, :, slot].cpu().double() - want_row[n, :C]).abs().max()) < tol
    assert int((kp.float().abs().sum(-1) > 0).sum()) == N                # nothing else was written
    if C % 16 == 0:           # the value pages in the order of the bf16 attention kernel's fragments
        vf = torch.zeros_like(vp)
        ops.latent_intake(dev(proj), dev(gain), 1e-5, cos, sin, qn, qf, kp, vf, table,
                          torch.tensor(seqs, dtype=torch.int32, device=DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
                          H, D, B, C, max(pos), v_fragments=True)
        assert torch.equal(vf, ops.latent_v_pages_to_kernel_order(vp))


# ----------------------------------------------------------------------------- whole models

def lengths(name):
    return {"P": [1, 2, 21, 64, 65, 150], "Q": [3, 70, 71, 129, 140], "R": [5, 64, 128, 200], "S": [1, 2, 3, 66, 90],
            "T": [2, 33, 34, 100], "U": [1, 8, 65, 80]}[name]


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S", "T", "U"]))
def test_whole_prompts(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        toks = tokens_for(name, n, 100 + i)
        s = eng.acquire()
        got = eng.step([(s, toks)], want="all")
        assert_logits_close(got, plain_logits(name, toks), dtype, f"{name} {dtype} {n} tokens whole", sharp=True)
        eng.release(s)
    eng.cache.check()


def test_the_residual_after_every_layer_in_float32():
    """The model's layers one after another: the residual rows that each leaves, read from the engine's own pass."""
    from synaptix_amd.parts import as_delta
    name = "P"
    toks = tokens_for(name, 70, 3)
    want = []
    plain_model(name).forward(toks, residuals=want)
    eng = engine(name, "float32")
    got = []
    for block in eng.model.blocks:
        inner = block.forward

        def spy(resid, pending, ctx, cache, owner=True, inner=inner):
            out = inner(resid, pending, ctx, cache, owner)
            got.append(resid.clone() + as_delta(out))
            return out
        block.forward = spy
    eng.step([(eng.acquire(), toks)], want="last")
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert float((a.cpu().double() - b).abs().max()) < 1e-4 * max(1.0, float(b.abs().max())), f"after layer {i}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_portions_of_several_sizes(name, dtype):
    """A prompt in portions of 2, 1, 3, 17, 64 and 2 tokens and the rest: every portion starts from the cache that
    the earlier ones left (inside a page, at a page's border, inside and beyond the first window)."""
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
    """Decoding long enough that every window passes over decoded tokens and over a page's border."""
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


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S", "T", "U"]))
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
    """Sequences of one and two tokens, and every position up to the window and a little more, one by one."""
    for name in ("P", "S"):
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
    """600 tokens one by one through the layers that keep every key and the one that keeps a window."""
    toks = tokens_for("P", 600, 5)
    want = plain_logits("P", toks)
    eng = engine("P", "float32", max_tokens=64 * 11)
    s = eng.acquire()
    got = [eng.step([(s, toks[:2])], want="all")]
    for t in toks[2:]:
        got.append(eng.step([(s, [t])], want="last"))
    assert_logits_close(torch.cat(got), want, "float32", "600 tokens one by one", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_pipeline(dtype):
    """Pipeline.generate_batch (the scheduler, slots, captured decode steps, the sampler) against greedy decoding with
    the plain model; in bfloat16 a token may differ where the two best logits are close, then the plain model's logits
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
    """Captured decode steps (three rows wide in a graph of four: one row is padding) with eager work of another
    sequence between the replays; every replay against the plain model."""
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
    spare page); portions of a prompt one after another, each from what the last one left."""
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
    from plain_kamivik import PlainKamivik

    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(CONFIGS["P"]))
    folder = str(tmp_path / "model")
    env = dict(os.environ, PYTHONPATH=ROOT)
    subprocess.run([sys.executable, "-m", "synaptix_amd", "random", str(cfg_file), folder, "--seed", "3"], check=True,
                   env=env, cwd=ROOT, timeout=300)
    plain = PlainKamivik.from_folder(folder)
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
