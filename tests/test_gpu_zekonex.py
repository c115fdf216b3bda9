"""Zekonex on the GPU against the plain model (`plain_zekonex`, NumPy float64): every kernel of its
own alone, each mixer alone in a one-layer model, then whole models of several tiny configurations
under every kind of schedule, in the 32-bit engine and in bfloat16 (held against the plain model
with bfloat16 storage as a yardstick)."""

import io
import json

import numpy as np
import pytest
import torch

import plain_zekonex as pz
import replay_util as ru
import tiny_zekonex as tz

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(values, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(values)).to(device=DEV, dtype=dtype)


def ints(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def rounded(values, dtype):
    """What the engine reads when `values` are stored in `dtype`, as float64."""
    return values.astype(np.float64) if dtype == "float32" else tz.bf16_round(values).astype(np.float64)


def tolerance(dtype, scale=1.0):
    return (2e-6 if dtype == "float32" else 1.2e-2) * scale


_ORACLES: dict = {}


def oracle(name, cfg, weights, tokens) -> ru.Oracle:
    key = (name, tuple(tokens))
    if key not in _ORACLES:
        wide = {k: v.astype(np.float64) for k, v in weights.items()}
        _ORACLES[key] = ru.Oracle(pz.logits(cfg, wide, tokens), pz.logits(cfg, wide, tokens, store=pz.bf16_round))
    return _ORACLES[key]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, block) in tz.CONFIGS.items():
        weights = tz.make_weights(cfg, seed=40 + len(out))
        out[name] = (cfg, block, weights, tz.write_model_dir(tmp_path_factory.mktemp("zekonex") / name, cfg, weights))
    return out


def runner_for(folder, dtype, block, pages=64, seats=4, graphs=True):
    from mini_infer_amd.engine import ModelRunner

    return ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block, max_concurrent=seats,
                                       cuda_graph=graphs)


# ---------------------------------------------------------------------------------------------
# each kernel alone
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [10, 64, 2500])
@pytest.mark.parametrize("parts", ["a", "ab", "ab+bias", "shift", "a+shift", "ab+bias+shift"])
def test_the_stream_update_and_the_norm_behind_it(dtype, width, parts):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width + len(parts))
    rows, scale, eps = 7, 0.3, 1e-5
    x = rng.standard_normal((rows, width)).astype(np.float32)
    a = rng.standard_normal((rows, width)).astype(np.float32) if "a" in parts else None
    b = rng.standard_normal((rows, width)).astype(np.float32) if "b" in parts.split("+")[0] and "ab" in parts else None
    bias = rng.standard_normal(width).astype(np.float32) if "bias" in parts else None
    shift = rng.standard_normal(width).astype(np.float32) if "shift" in parts else None
    weight = rng.uniform(0.5, 1.5, width).astype(np.float32)
    total = np.zeros((rows, width))
    for part in (a, b):
        if part is not None:
            total = total + rounded(part, dtype)
    if bias is not None:
        total = total + bias
    new = x.astype(np.float64) + scale * total + (0 if shift is None else shift.astype(np.float64))
    normed = new / np.sqrt((new * new).mean(1, keepdims=True) + eps) * rounded(weight, dtype)
    update = ops.StreamUpdate(None if a is None else dev(a, TORCH[dtype]), None if b is None else dev(b, TORCH[dtype]),
                              None if bias is None else dev(bias), None if shift is None else dev(shift), scale)
    stream = dev(x)
    out = ops.stream_update_norm(update, stream, dev(weight, TORCH[dtype]), eps)
    np.testing.assert_allclose(stream.cpu().numpy(), new, rtol=0, atol=2e-6)
    np.testing.assert_allclose(out.float().cpu().numpy(), normed, rtol=0, atol=tolerance(dtype, 4))
    # at chosen rows only: the stream stays as it was
    stream = dev(x)
    some = ops.stream_update_norm(update, stream, dev(weight, TORCH[dtype]), eps, rows=ints([5, 0]))
    np.testing.assert_array_equal(stream.cpu().numpy(), x)
    np.testing.assert_allclose(some.float().cpu().numpy(), normed[[5, 0]], rtol=0, atol=tolerance(dtype, 4))
    # what anything that knows no such update would add instead
    np.testing.assert_allclose(np.broadcast_to(update.finish().cpu().numpy(), x.shape), new - x, rtol=0, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter, limit", [(5, 0.7), (64, 1.5), (300, 3.0)])
def test_the_clamped_gated_activation(dtype, inter, limit):
    from mini_infer_amd import ops

    rng = np.random.default_rng(inter)
    rows = rng.standard_normal((9, 2 * inter)).astype(np.float32) * 2.5  # (well past the limit on both sides)
    bias = rng.standard_normal(2 * inter).astype(np.float32)
    z = rounded(rows, dtype) + bias
    g, u = np.minimum(z[:, :inter], limit), np.clip(z[:, inter:], -limit, limit)
    want = g / (1 + np.exp(-1.702 * g)) * (u + 1)
    got = ops.clamped_glu(dev(rows, TORCH[dtype]), dev(bias), limit, 1.702)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=0, atol=tolerance(dtype, 2 * limit * (limit + 1)))
    assert (np.abs(z[:, :inter]) > limit).any() and (z[:, inter:] < -limit).any()


@pytest.mark.parametrize("rows, inter, k", [(1, 24, 64), (8, 70, 256), (16, 320, 256), (17, 48, 96), (32, 130, 512), (33, 24, 64)])
def test_gated_product_with_biases_clamps_and_activation_in_its_last_step(rows, inter, k):
    """Few bfloat16 rows: one kernel, bit-equal to the product followed by the activation's kernel
    (33 rows: the two in turn, on both sides)."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(rows * inter)
    x = dev(rng.standard_normal((rows, k)).astype(np.float32), torch.bfloat16)
    weight = dev((rng.standard_normal((2 * inter, k)) / np.sqrt(k) * 2.5).astype(np.float32), torch.bfloat16)
    bias = dev(rng.standard_normal(2 * inter).astype(np.float32))
    fused = ops.linear_clamped_glu(x, weight, bias, 1.3, 1.702)
    in_turn = ops.clamped_glu(ops.linear(x, weight), bias, 1.3, 1.702)
    assert torch.equal(fused, in_turn)
    z = (x.double() @ weight.double().T).cpu().numpy() + bias.cpu().numpy()
    g, u = np.minimum(z[:, :inter], 1.3), np.clip(z[:, inter:], -1.3, 1.3)
    np.testing.assert_allclose(fused.float().cpu().numpy(), g / (1 + np.exp(-1.702 * g)) * (u + 1), rtol=0, atol=4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels, taps", [(10, 1), (70, 2), (256, 4), (33, 7)])
def test_the_short_convolution_carries_each_requests_tail(dtype, channels, taps):
    """Five steps over four requests of unequal length, among them portions shorter than the tail,
    a request that brings nothing, and one that starts later in a slot of its own."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(channels)
    weight = (rng.standard_normal((channels, taps)) * 0.6).astype(np.float32)
    tails = torch.zeros((6, max(taps - 1, 0), channels), dtype=TORCH[dtype], device=DEV)
    plain = {slot: np.zeros((taps - 1, channels)) for slot in range(5)}
    # (steps of up to 64 rows run as one launch, a thread walking a request's rows; longer ones as two)
    for step, lengths in enumerate([(1, 9, 0, 2), (2, 1, 5, 1), (80, 1, 1, 3), (1, 1, 0, 1), (30, 2, 70, 1)]):
        slots = [3, 0, 4, 1]
        x = rng.standard_normal((sum(lengths), channels + 5)).astype(np.float32)  # (the projection's rows are wider)
        cu = np.concatenate([[0], np.cumsum(lengths)])
        request_of = np.repeat(np.arange(4), lengths)
        got = ops.short_conv(dev(x, TORCH[dtype]), channels, dev(weight), tails, ints(cu), ints(slots), ints(request_of))
        for b, slot in enumerate(slots):
            z = rounded(x[cu[b]:cu[b + 1], :channels], dtype)
            y, plain[slot] = pz.short_convolution(z, weight.astype(np.float64), plain[slot])
            np.testing.assert_allclose(got[cu[b]:cu[b + 1]].float().cpu().numpy(), pz.silu(y), rtol=0,
                                       atol=tolerance(dtype, 4), err_msg=f"step {step} request {b}")
            if taps > 1:
                np.testing.assert_array_equal(tails[slot].float().cpu().numpy(), plain[slot])


def paged(rows: np.ndarray, page_size: int, order: list[int], dtype) -> torch.Tensor:
    """[tokens, heads, dim] laid into pages [num_pages, heads, page_size, dim], page i of the
    request at page id order[i]."""
    tokens, heads, dim = rows.shape
    pages = np.zeros((max(order) + 1, heads, page_size, dim), dtype=np.float32)
    for t in range(tokens):
        pages[order[t // page_size], :, t % page_size] = rows[t]
    return dev(pages, TORCH[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page", [(4, 2, 16, 24, 8), (3, 3, 10, 6, 4), (8, 1, 64, 64, 16), (5, 1, 130, 66, 16),
                                                               (8, 2, 128, 128, 16), (4, 4, 32, 32, 32)])
def test_attention_with_a_sink_and_values_of_another_width(dtype, heads, kv_heads, dim, vdim, page):
    """One request of 333 keys in scattered pages, queries at its last 5 positions.  Head 0's
    last query is made to single out key 3, far back; head 1's scores are all far below the
    sink's, so the sink takes nearly all the weight; the rest are random."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim)
    keys_n, queries_n, scale = 333, 5, 0.5
    k = rng.standard_normal((keys_n, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((keys_n, kv_heads, vdim)).astype(np.float32)
    q = rng.standard_normal((queries_n, heads, dim)).astype(np.float32)
    q[-1, 0] = 6.0 * k[3, 0] / np.linalg.norm(k[3, 0])
    k[3, 0] *= 3.0
    if heads > 1:
        q[:, 1] = -4.0 * np.abs(q[:, 1])
        k[:, 1 // (heads // kv_heads)] = np.abs(k[:, 1 // (heads // kv_heads)]) + 0.5
        if 1 // (heads // kv_heads) == 0:
            q[-1, 0] = 6.0 * k[3, 0] / np.linalg.norm(k[3, 0])
    order = list(rng.permutation(-(-keys_n // page) + 3))[: -(-keys_n // page)]
    positions = np.arange(keys_n - queries_n, keys_n)
    got = ops.paged_attention(
        dev(q.reshape(queries_n, -1), TORCH[dtype]), paged(k, page, order, dtype), paged(v, page, order, dtype),
        ints(order).view(1, -1), ints([0] * queries_n), ints(positions), ints([0, queries_n]), [0, queries_n],
        q_heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale, window=None, max_seq_len=keys_n, v_head_dim=vdim,
        sink_logit=0.0,
    ).float().cpu().numpy().reshape(queries_n, heads, vdim)
    kq, vq, qq = rounded(k, dtype), rounded(v, dtype), rounded(q, dtype)
    group = heads // kv_heads
    want = np.zeros((queries_n, heads, vdim))
    weight_on_3 = sunk = None
    for i, p in enumerate(positions):
        for a in range(heads):
            s = kq[: p + 1, a // group] @ qq[i, a] * scale
            e = np.exp(s)
            want[i, a] = e @ vq[: p + 1, a // group] / (1.0 + e.sum())
            if i == queries_n - 1 and a == 0:
                weight_on_3 = e[3] / (1.0 + e.sum())
            if a == 1:
                sunk = 1.0 / (1.0 + e.sum())
    np.testing.assert_allclose(got, want, rtol=0, atol=tolerance(dtype, 4))
    assert weight_on_3 > 0.9  # the far key is what the answer is made of
    if ops.mfma_attention_supported(TORCH[dtype], dim, page) and vdim == dim:
        # the matrix-core kernel (values transposed inside a page) knows the sink too: the queries as a
        # prompt's last portion, and the last one alone as a decoded token (keys cut into ranges)
        v_t = paged(v, page, order, dtype).transpose(2, 3).contiguous()
        for rows in (slice(0, queries_n), slice(queries_n - 1, queries_n)):
            n = rows.stop - rows.start
            fast = ops.paged_attention(
                dev(q[rows].reshape(n, -1), TORCH[dtype]), paged(k, page, order, dtype), v_t, ints(order).view(1, -1), ints([0] * n),
                ints(positions[rows]), ints([0, n]), [0, n], q_heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale,
                window=None, max_seq_len=keys_n, v_transposed=True, sink_logit=0.0,
            ).float().cpu().numpy().reshape(n, heads, vdim)
            np.testing.assert_allclose(fast, want[rows], rtol=0, atol=tolerance(dtype, 4))
    if heads > 1:
        assert sunk > 0.99 and np.abs(want[:, 1]).max() < 0.05 < np.abs(vq).mean()  # a sink left out would show


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot, rank, page", [(3, 10, 6, 22, 8), (4, 32, 32, 96, 16), (2, 6, 2, 18, 4)])
def test_latent_rows_and_rotated_query_parts(dtype, heads, dim, rot, rank, page):
    from mini_infer_amd import ops

    rng = np.random.default_rng(rank)
    tokens, eps, base = 11, 1e-5, 50.0
    head_width, c_col = dim + rot, heads * (dim + rot)
    proj = rng.standard_normal((tokens, c_col + rank + rot + 3)).astype(np.float32)
    weight = rng.uniform(0.5, 1.5, rank).astype(np.float32)
    positions = np.arange(40, 40 + tokens)
    angles = positions[:, None] * base ** (-2.0 * np.arange(rot // 2) / rot)
    slots = rng.permutation(5 * page)[:tokens]
    slots[4] = -1  # (a padding row of a recorded step writes nowhere)
    pages = torch.zeros((5, 1, page, rank + rot), dtype=TORCH[dtype], device=DEV)
    queries = torch.zeros((tokens, heads * (rank + rot)), dtype=TORCH[dtype], device=DEV)
    ops.latent_prepare(dev(proj, TORCH[dtype]), dev(np.cos(angles)), dev(np.sin(angles)), dev(weight), ints(slots), pages, queries,
                       heads=heads, q_head_width=head_width, q_rot_at=dim, c_col=c_col, rank=rank, rot=rot, eps=eps)
    p = rounded(proj, dtype)
    flat = pages.float().cpu().numpy().reshape(5 * page, rank + rot)
    got_q = queries.float().cpu().numpy().reshape(tokens, heads, rank + rot)
    for t in range(tokens):
        for a in range(heads):
            turned = pz.rotate_pairs(p[t, a * head_width + dim: (a + 1) * head_width], int(positions[t]), base, rot)
            np.testing.assert_allclose(got_q[t, a, rank:], turned, rtol=0, atol=tolerance(dtype, 4))
        if slots[t] < 0:
            continue
        row = np.concatenate([pz.rms_norm(p[t, c_col: c_col + rank], weight.astype(np.float64), eps),
                              pz.rotate_pairs(p[t, c_col + rank: c_col + rank + rot], int(positions[t]), base, rot)])
        np.testing.assert_allclose(flat[slots[t]], row, rtol=0, atol=tolerance(dtype, 4))
    assert np.count_nonzero(np.abs(flat).sum(1)) == tokens - 1


# ---------------------------------------------------------------------------------------------
# each mixer alone: a model of one layer without a feed-forward
# ---------------------------------------------------------------------------------------------

ALONE = {
    "attention": tz.attention(4, 2, 16, 24, 0.8, rot=(100.0, 8)),
    "attention_unrotated_one_kv_head": tz.attention(6, 1, 10, 4, 0.9),
    "latent": tz.latent(3, 10, 6, 14, 22, 0.8, 50.0),
    "latent_one_head": tz.latent(1, 32, 32, 64, 64, 0.4, 10000.0),
    "delta": tz.delta(4, 2, 12, 20, 3),
    "delta_odd_sizes_one_tap": tz.delta(3, 3, 7, 9, 1),
    "delta_large_heads": tz.delta(1, 1, 132, 80, 4),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", sorted(ALONE))
def test_each_mixer_alone_whole_and_token_by_token(tmp_path, dtype, mixer):
    from mini_infer_amd.engine import StepEntry

    cfg = tz.config(90, 48, [ALONE[mixer]], scale=2.0, eps=1e-5, mult=0.8)
    weights = tz.make_weights(cfg, seed=len(mixer))
    folder = tz.write_model_dir(tmp_path / "m", cfg, weights)
    tokens = tz.random_tokens(cfg, 45, seed=9)
    want = oracle(mixer, cfg, weights, tokens)
    runner = runner_for(folder, dtype, 8, pages=12, seats=2)
    whole = runner.step([StepEntry("w", tokens, list(range(45)))]).cpu().numpy()
    ru.assert_close(whole, want, dtype, f"{mixer} whole")
    one_by_one = np.concatenate([runner.step([StepEntry("d", [t], [0])]).cpu().numpy() for t in tokens])
    ru.assert_close(one_by_one, want, dtype, f"{mixer} token by token")


# ---------------------------------------------------------------------------------------------
# whole models under every kind of schedule
# ---------------------------------------------------------------------------------------------

LENGTHS = {"A": (70, 41, 9, 33, 58, 1), "B": (45, 64, 17, 2, 39), "C": (130, 40, 77, 5), "D": (50, 21, 36, 3, 44),
           "E": (90, 35, 66, 3)}


def requests_of(name, cfg):
    return {f"{name}{i}": tz.random_tokens(cfg, n, seed=100 * len(name) + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(tz.CONFIGS))
@pytest.mark.parametrize("family", ["whole", "decode", "portions", "mixed"])
def test_logits_do_not_depend_on_the_schedule(folders, name, dtype, family):
    """Whole prompts; a prompt and then its last tokens one by one; portions down to two tokens;
    up to four live requests of unequal length in one batch, in a pool so small that pages and
    state slots are used again.  Each request is held against itself alone."""
    cfg, block, weights, folder = folders[name]
    requests = requests_of(name, cfg)
    schedule = {
        "whole": lambda: ru.schedule_whole(requests),
        "decode": lambda: ru.schedule_prefill_then_decode(requests, tail=36),
        "portions": lambda: ru.schedule_portions(requests, seed=3),
        "mixed": lambda: ru.schedule_mixed(requests, seed=5, max_live=4, tail=12),
    }[family]()
    pages = ru.peak_pages(requests, schedule, block)
    runner = runner_for(folder, dtype, block, pages=pages, seats=4 if family == "mixed" else 1)
    got = ru.run_schedule(runner, requests, schedule)
    for rid, tokens in requests.items():
        ru.assert_close(got[rid], oracle(name, cfg, weights, tokens), dtype, f"{name} {family} {rid}")
    runner.cache.check()
    assert runner.cache.states.num_free == runner.cache.states.max_requests
    assert runner.num_free_blocks() == pages


def test_prompts_that_come_whole_write_keys_and_values_out_per_head(folders, monkeypatch):
    """bfloat16, a latent attention layer whose head sizes the matrix-core kernel takes: a step in
    which every request begins takes the expanded form (two prompts side by side, neither filling
    its last page), any other step the folded one; both agree with the plain model."""
    from mini_infer_amd.engine import StepEntry
    from mini_infer_amd.parts.latent_attention import LatentAttention

    cfg, block, weights, folder = folders["C"]
    calls = []
    original = LatentAttention._forward_expanded
    monkeypatch.setattr(LatentAttention, "_forward_expanded", lambda self, *a, **k: (calls.append(1), original(self, *a, **k))[1])
    runner = runner_for(folder, "bfloat16", block, pages=24, seats=2)
    first, second = tz.random_tokens(cfg, 101, seed=5), tz.random_tokens(cfg, 70, seed=6)
    both = runner.step([StepEntry("p", first[:90], list(range(90))), StepEntry("q", second, list(range(70)))]).cpu().numpy()
    assert len(calls) == 1  # (one latent attention layer in this configuration)
    rest = runner.step([StepEntry("p", first[90:], list(range(11)))]).cpu().numpy()
    assert len(calls) == 1  # a later portion reads the cache: folded
    ru.assert_close(np.concatenate([both[:90], rest]), oracle("C", cfg, weights, first), "bfloat16", "whole then a portion")
    ru.assert_close(both[90:], oracle("C", cfg, weights, second), "bfloat16", "beside it")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_and_pages_used_again_start_clean(folders, dtype):
    """One seat, pages for one request: the second request gets the first one's slot (recurrent
    state and convolution tails of every pass) and pages."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["A"]
    first, second = tz.random_tokens(cfg, 30, seed=1), tz.random_tokens(cfg, 26, seed=2)
    runner = runner_for(folder, dtype, block, pages=2, seats=1)
    runner.step([StepEntry("a", first, [])])
    slot = runner.cache.state_slot("a")
    runner.free_request("a")
    got = runner.step([StepEntry("b", second[:2], [0, 1])]).cpu().numpy()
    assert runner.cache.state_slot("b") == slot
    got = np.concatenate([got, runner.step([StepEntry("b", second[2:], list(range(24)))]).cpu().numpy()])
    ru.assert_close(got, oracle("A", cfg, weights, second), dtype, "second owner of a slot")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds_and_long_decoding_through_recorded_steps(folders, dtype):
    """Two requests decoded side by side for 150 steps after prompts of 210 and 7 tokens, across
    many page borders; the single-token steps are replayed graphs."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["A"]
    requests = {"x": tz.random_tokens(cfg, 360, seed=31), "y": tz.random_tokens(cfg, 157, seed=32)}
    runner = runner_for(folder, dtype, block, pages=34, seats=2)
    got = {rid: [] for rid in requests}
    both = runner.step([StepEntry("x", requests["x"][:210], list(range(210))), StepEntry("y", requests["y"][:7], list(range(7)))]).cpu().numpy()
    got["x"].append(both[:210])
    got["y"].append(both[210:])
    for k in range(150):
        logits = runner.step([StepEntry("x", [requests["x"][210 + k]], [0]), StepEntry("y", [requests["y"][7 + k]], [0])]).cpu().numpy()
        got["x"].append(logits[:1])
        got["y"].append(logits[1:])
    assert runner.decode_graphs is not None and runner.decode_graphs.replays == 150
    for rid, tokens in requests.items():
        ru.assert_close(np.concatenate(got[rid]), oracle("A", cfg, weights, tokens), dtype, f"long decoding {rid}")


def test_a_lost_state_a_sink_or_a_pass_vector_left_out_would_show(folders):
    """The tiny weights make every mechanism matter: the plain model with one of them switched
    off is far from the plain model."""
    cfg, block, weights, _ = folders["A"]
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    tokens = tz.random_tokens(cfg, 40, seed=77)
    base = pz.logits(cfg, wide, tokens)

    def far(other) -> bool:
        return np.abs(other - base).max() > 100 * ru.FP32_TOL

    model = pz.PlainZekonex(cfg, wide)
    memory: dict = {}
    head = model.forward(tokens[:20], memory)
    for run, kept in memory.items():  # the recurrent state of one pass is lost between two portions
        if isinstance(kept, dict) and "S" in kept:
            lost = {k: (dict(v, S=np.zeros_like(v["S"])) if k == run else v) for k, v in memory.items()}
            lost = {k: (dict(v) if isinstance(v, dict) else v) for k, v in lost.items()}
            assert far(np.concatenate([head, model.forward(tokens[20:], lost)])), f"state of run {run}"
            break
    no_steps = dict(wide, **{"loop.step": np.zeros_like(wide["loop.step"])})
    assert far(pz.logits(cfg, no_steps, tokens))
    same_steps = dict(wide, **{"loop.step": np.repeat(wide["loop.step"][:1], 3, axis=0)})
    assert far(pz.logits(cfg, same_steps, tokens))
    original = pz.sink_attention

    def without_sink(h, w, m, first=0, past=None, store=pz.keep):
        """The same attention with an ordinary softmax (a sink so low that it takes nothing)."""
        heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        count = h.shape[0]
        q = (h @ w["q"].T).reshape(count, heads, dim)
        k = (h @ w["k"].T).reshape(count, groups, dim)
        v = (h @ w["v"].T).reshape(count, groups, vdim)
        for t in range(count):
            q[t] = [pz.rotate_pairs(row, first + t, m["rot"]["base"], m["rot"]["dims"]) for row in q[t]]
            k[t] = [pz.rotate_pairs(row, first + t, m["rot"]["base"], m["rot"]["dims"]) for row in k[t]]
        out = np.zeros((count, heads, vdim))
        for t in range(count):
            for a in range(heads):
                s = k[: t + 1, a // (heads // groups)] @ q[t, a] * m["scale"]
                e = np.exp(s - s.max())
                out[t, a] = e @ v[: t + 1, a // (heads // groups)] / e.sum()
        return out.reshape(count, heads * vdim) @ w["o"].T

    try:
        pz.sink_attention = without_sink
        assert far(pz.logits(cfg, wide, tokens))
    finally:
        pz.sink_attention = original


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_llm_and_the_scheduler(folders, name):
    """Five prompts for two seats, prompts cut into portions of 8 under a 20-token budget: every
    generated token is the plain model's greedy choice."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = folders[name]
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    lengths, new_tokens = (5, 19, 33, 2, 11), 9
    prompts = [tz.random_tokens(cfg, n, seed=300 + n) for n in lengths]
    llm = LLM(folder, dtype="float32", num_blocks=12, block_size=block, max_concurrent=2, max_num_batched_tokens=20, chunk_size=8)
    results = llm.generate(prompts, max_tokens=new_tokens)
    for prompt, result in zip(prompts, results):
        sequence = list(prompt)
        for _ in range(new_tokens):
            sequence.append(pz.greedy(pz.logits(cfg, wide, sequence)[-1]))
        assert result.tokens == sequence[len(prompt):] and result.finish_reason == "length"
    assert llm.runner.cache.states.num_free == 2
    llm.runner.cache.check()


def test_a_norm_that_knows_no_stream_update_is_handed_the_finished_sum(folders):
    """The parallel block leaves its add to the next norm as an update not made yet.  `rms_norm` makes it
    in its own launch; a norm of another kind (here the one-gain norm as final norm) gets the finished
    sum instead.  With a weight that is the gain in every column the two models are one function."""
    import dataclasses

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.models.decoder import DecoderModel
    from mini_infer_amd.models.zekonex import ZekonexConfig, zekonex_spec
    from mini_infer_amd.weights.loader import load_state_dict

    cfg, block, weights, _ = folders["A"]
    spec = zekonex_spec(ZekonexConfig.from_dict(cfg))
    one_gain = dataclasses.replace(spec, final_norm={"kind": "scalar_rms_norm", "hidden_size": cfg["width"],
                                                     "eps": cfg["norm"]["eps"], "name": "norm"})
    tensors = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in weights.items()}
    tokens = tz.random_tokens(cfg, 37, seed=8)
    got = []
    for model_spec, final in ((spec, torch.full((cfg["width"],), 0.75)), (one_gain, torch.tensor(0.75))):
        model = DecoderModel(model_spec, torch.float32, DEV)
        load_state_dict(model, dict(tensors, **{"final.norm": final}))
        runner = ModelRunner(model, None, num_blocks=4, block_size=block, max_concurrent=1)
        first = runner.step([StepEntry("r", tokens[:30], list(range(30)))]).cpu().numpy()
        rest = [runner.step([StepEntry("r", [t], [0])]).cpu().numpy() for t in tokens[30:]]
        got.append(np.concatenate([first, *rest]))
    np.testing.assert_allclose(got[1], got[0], rtol=0, atol=2e-5)
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    wide["final.norm"] = np.full(cfg["width"], 0.75)
    ru.assert_close(got[0], pz.logits(cfg, wide, tokens), "float32", "weight of one value")


def test_the_command_line_writes_random_weights_and_generates_greedily_and_by_seeded_sampling(tmp_path, capsys):
    """`random-weights` from a config.json, then `generate`: greedy twice the same, sampled with one seed
    twice the same and (at this temperature) different from greedy."""
    from mini_infer_amd.__main__ import main

    cfg, block = tz.CONFIGS["A"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert main(["random-weights", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(tmp_path / "m"),
                 "--std", "0.3", "--norm-jitter", "0.1"]) == 0
    capsys.readouterr()

    def generate(*extra):
        assert main(["generate", "--model", str(tmp_path / "m"), "--prompt-ids", "5 9 100 3 77", "--prompt-ids", "1,2",
                     "--max-tokens", "12", "--num-blocks", "16", "--block-size", str(block), "--max-concurrent", "2",
                     "--ignore-eos", *extra]) == 0
        lines = [json.loads(line) for line in capsys.readouterr().out.strip().splitlines()]
        assert [line["prompt_tokens"] for line in lines] == [5, 2] and all(len(line["tokens"]) == 12 for line in lines)
        return [line["tokens"] for line in lines]

    greedy = generate()
    assert generate() == greedy
    sampled = generate("--temperature", "1.5", "--top-k", "40", "--top-p", "0.95", "--seed", "11")
    assert generate("--temperature", "1.5", "--top-k", "40", "--top-p", "0.95", "--seed", "11") == sampled
    assert sampled != greedy and all(0 <= t < cfg["vocab"] for tokens in sampled for t in tokens)


def test_the_replay_program_runs_a_trace_of_this_design(folders, tmp_path):
    from mini_infer_amd.engine import replay, trace

    cfg, block, weights, folder = folders["B"]
    requests = {f"t{i}": tz.random_tokens(cfg, n, seed=i) for i, n in enumerate((70, 41, 9, 33, 58))}
    schedule = trace.make_schedule("mixed", requests, seed=1, tail=10)
    lines = trace.to_trace_lines(requests, schedule)
    limit = trace.peak_pages(requests, schedule, 64) * 64
    args = replay.build_parser().parse_args(["--model", str(folder), "--dtype", "float32", "--out", str(tmp_path / "out"),
                                             "--max-tokens", str(limit)])
    said = io.StringIO()
    assert replay.run(args, lines=lines, out=said) == 0
    assert said.getvalue().split() == [w for n in range(len(lines)) for w in ("done", str(n))]
    fed = {rid: 0 for rid in requests}
    for number, line in enumerate(lines):
        step = json.loads(line)
        got = np.fromfile(tmp_path / "out" / f"{number}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        at = 0
        for entry in step["entries"]:
            n, rid = len(entry["tokens"]), entry["id"]
            want = oracle("B", cfg, weights, requests[rid])[slice(fed[rid], fed[rid] + n)]
            ru.assert_close(got[at: at + n], want, "float32", f"trace step {number} {rid}")
            fed[rid] += n
            at += n
