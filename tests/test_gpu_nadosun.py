"""Nadosun on the GPU against the plain model (`plain_nadosun`, NumPy float64): every kernel of its
own alone, then whole models of several tiny configurations under every kind of schedule, in the
32-bit engine and in bfloat16 (held against the plain model with bfloat16 storage as a yardstick)."""

import io
import json

import numpy as np
import pytest
import torch

import plain_nadosun as pn
import replay_util as ru
import tiny_nadosun as tn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(values, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(values)).to(device=DEV, dtype=dtype)


def rounded(values, dtype):
    """What the engine reads when `values` are stored in `dtype`, as float64."""
    return values.astype(np.float64) if dtype == "float32" else tn.bf16_round(values).astype(np.float64)


def tolerance(dtype, scale=1.0):
    return (2e-6 if dtype == "float32" else 1.2e-2) * scale


_ORACLES: dict = {}


def oracle(name, cfg, weights, tokens) -> ru.Oracle:
    key = (name, tuple(tokens))
    if key not in _ORACLES:
        _ORACLES[key] = ru.Oracle(pn.logits(cfg, weights, tokens), pn.logits(cfg, weights, tokens, store=pn.bf16_round))
    return _ORACLES[key]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, block) in tn.CONFIGS.items():
        weights = tn.make_weights(cfg, seed=20 + len(out))
        out[name] = (cfg, block, weights, tn.write_model_dir(tmp_path_factory.mktemp("nadosun") / name, cfg, weights))
    return out


def runner_for(folder, dtype, block, pages=64, seats=4, graphs=True):
    from mini_infer_amd.engine import ModelRunner

    return ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block, max_concurrent=seats,
                                       cuda_graph=graphs)


# ---------------------------------------------------------------------------------------------
# each kernel alone
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [7, 64, 90])
def test_embedding_with_scale_and_sinusoid(dtype, width):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width)
    table = rounded(rng.standard_normal((40, width)).astype(np.float32), "bfloat16")
    ids = rng.integers(0, 40, size=9)
    positions = np.array([0, 1, 2, 15, 16, 17, 63, 1000, 4099])
    freq = dev(10000.0 ** (-2.0 * np.arange((width + 1) // 2) / width), torch.float64)
    stream, cast = ops.embed_sinusoid(dev(table, TORCH[dtype]), dev(ids, torch.int32), dev(positions, torch.int32), freq,
                                      2.5, want_cast=dtype == "bfloat16")
    want = table[ids] * 2.5 + pn.sinusoid(positions, width)
    # (the bfloat16 engine takes the angle in float32: 4099 * 2^-24 radians off at most)
    assert np.abs(stream.cpu().numpy() - want).max() < (3e-6 if dtype == "float32" else 6e-4)
    if cast is not None:
        assert torch.equal(cast, stream.bfloat16())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_gain, with_scale", [(True, True), (True, False), (False, True)])
def test_norm_on_a_sublayers_output_adds_into_the_stream(dtype, with_gain, with_scale):
    from mini_infer_amd import ops

    rng = np.random.default_rng(4)
    for hidden in (5, 96, 1030):
        y = rounded(3.0 * rng.standard_normal((6, hidden)).astype(np.float32), dtype)
        stream = rng.standard_normal((6, hidden)).astype(np.float32)
        gain, scale = np.float32(1.37), rng.uniform(0.5, 1.5, hidden).astype(np.float32)
        want = stream + pn.rms(y, 1e-5) * (gain if with_gain else 1.0) * (scale if with_scale else 1.0)
        res = dev(stream)
        cast = ops.norm_scale_add(dev(y, TORCH[dtype]), res, dev(np.array([gain])) if with_gain else None,
                                  dev(scale) if with_scale else None, 1e-5, want_cast=True)
        assert np.abs(res.cpu().numpy() - want).max() < 2e-6 * max(1.0, np.abs(want).max())
        assert torch.equal(cast, res.to(TORCH[dtype]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [70, 72, 192])  # (columns in fours and whole tiles of 64, or neither)
@pytest.mark.parametrize("lengths, max_rows", [((1, 1, 1), 1), ((5, 0, 17, 2), 17), ((300, 131, 64, 1), 300), ((129,), None),
                                               ((129, 0, 200), 200)])
def test_gated_recurrence_over_unequal_requests_with_carried_state(dtype, lengths, max_rows, width):
    """Rows of several requests in one launch, one of them without rows, one whose slot is nobody's;
    the state that comes in is not zero, and what goes out is what the next portion starts from."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(sum(lengths))
    slots = 6
    total = sum(lengths)
    zxg = rounded(2.0 * rng.standard_normal((total, 3 * width)).astype(np.float32), dtype)
    bz, bx = rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    state = rng.standard_normal((slots + 1, width)).astype(np.float32)
    owners = [3, 0, -1, 5][: len(lengths)]
    cu = np.concatenate([[0], np.cumsum(lengths)])
    # (state rows of different slots lie further apart than their own width, as in the engine's state buffer)
    buffer = torch.full((slots + 1, width + 26), 9.0, device=DEV)
    state_d = buffer[:, 3 : 3 + width]
    state_d.copy_(dev(state))
    got = ops.gated_scan(dev(zxg, TORCH[dtype]), dev(bz), dev(bx), state_d, dev(cu, torch.int32), dev(np.array(owners), torch.int32),
                         max_rows).float().cpu().numpy()
    after = state_d.cpu().numpy()
    touched = set()
    for b, n in enumerate(lengths):
        if n == 0:
            continue  # a request without rows leaves its state alone
        row = owners[b] if owners[b] >= 0 else slots
        rows = zxg[cu[b] : cu[b + 1]]
        want, last = pn.gated_recurrence(rows[:, :width] + bz, rows[:, width : 2 * width] + bx, rows[:, 2 * width :], state[row])
        touched.add(row)
        assert np.abs(got[cu[b] : cu[b + 1]] - rounded(want.astype(np.float32), dtype)).max() < tolerance(dtype, 4.0)
        assert np.abs(after[row] - last).max() < 2e-5
    for row in set(range(slots + 1)) - touched:
        assert np.array_equal(after[row], state[row])
    assert bool((buffer[:, :3] == 9.0).all()) and bool((buffer[:, 3 + width :] == 9.0).all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transposed", [False, True])
def test_whole_projection_norm_and_cache_write(dtype, transposed):
    from mini_infer_amd import ops

    rng = np.random.default_rng(8)
    tokens, heads, kv_heads, dim, page, pages = 7, 3, 2, 10, 4, 5
    q_width, k_width = heads * dim, kv_heads * dim
    qk = rounded(rng.standard_normal((tokens, q_width + k_width)).astype(np.float32) * 2, dtype)
    qw, kw = rng.uniform(0.5, 1.5, q_width).astype(np.float32), rng.uniform(0.5, 1.5, k_width).astype(np.float32)
    slots = np.array([17, 2, -1, 3, 8, 19, 0])
    k_pages = torch.zeros((pages, kv_heads, page, dim), dtype=TORCH[dtype], device=DEV)
    v_pages = torch.zeros((pages, kv_heads, dim, page) if transposed else (pages, kv_heads, page, dim), dtype=TORCH[dtype], device=DEV)
    qk_d = dev(qk, TORCH[dtype])
    ops.qk_norm_kv_write(qk_d, dev(qw), dev(kw), dev(slots, torch.int32), k_pages, v_pages, q_width=q_width, kv_heads=kv_heads,
                         head_dim=dim, eps=1e-5, v_transposed=transposed)
    tol = tolerance(dtype, 3.0)
    assert np.abs(qk_d[:, :q_width].float().cpu().numpy() - pn.rms(qk[:, :q_width], 1e-5) * qw).max() < tol
    want_k = pn.rms(qk[:, q_width:], 1e-5) * kw
    keys = k_pages.float().cpu().numpy()
    values = v_pages.float().cpu().numpy()
    if transposed:
        values = values.transpose(0, 1, 3, 2)
    written = np.zeros((pages, page), dtype=bool)
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        written[slot // page, slot % page] = True
        for h in range(kv_heads):
            assert np.abs(keys[slot // page, h, slot % page] - want_k[t, h * dim : (h + 1) * dim]).max() < tol
            assert np.array_equal(values[slot // page, h, slot % page], qk[t, q_width + h * dim : q_width + (h + 1) * dim].astype(np.float32))
    unwritten = ~written  # a negative slot writes nowhere
    assert not keys.transpose(0, 2, 1, 3)[unwritten].any() and not values.transpose(0, 2, 1, 3)[unwritten].any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_poly_norm_activation(dtype):
    from mini_infer_amd import ops

    rng = np.random.default_rng(2)
    coefficients = np.array([0.8, -0.6, 0.3, 0.15], dtype=np.float32)
    for width in (3, 130, 2048):
        z = rounded(1.5 * rng.standard_normal((5, width)).astype(np.float32), dtype)
        got = ops.poly_norm(dev(z, TORCH[dtype]), dev(coefficients), 1e-6).float().cpu().numpy()
        want = pn.poly_norm(z, coefficients, 1e-6)
        assert np.abs(got - want).max() < tolerance(dtype, np.abs(want).max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_rows_of_a_shared_table(dtype):
    from mini_infer_amd import ops

    rng = np.random.default_rng(6)
    gate = rounded(2.0 * rng.standard_normal((9, 5)).astype(np.float32), dtype)
    table = rounded(rng.standard_normal((30, 20)).astype(np.float32), dtype)
    ids = rng.integers(0, 30, size=9)
    got = ops.gated_table_rows(dev(gate, TORCH[dtype]), dev(table, TORCH[dtype]), dev(ids, torch.int32), 10).float().cpu().numpy()
    want = pn.gelu_tanh(gate) * table[ids, 10:15]
    assert np.abs(got - want).max() < tolerance(dtype, np.abs(want).max())


@pytest.mark.parametrize("rows, features, k", [(1, 24, 64), (8, 26, 256), (16, 128, 96), (17, 24, 64)])
def test_gate_product_with_activation_and_gather_in_its_last_step(rows, features, k):
    """Few bfloat16 rows run as one kernel; its values are those of the product followed by the
    activation kernel, bit for bit (17 rows: the two-kernel route itself)."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(rows + features)
    x = tn.bf16_round(rng.standard_normal((rows, k)).astype(np.float32))
    weight = tn.bf16_round((rng.standard_normal((features, k)) / np.sqrt(k)).astype(np.float32) * 2)
    table = tn.bf16_round(rng.standard_normal((21, 3 * features + 5)).astype(np.float32))
    ids = rng.integers(0, 21, size=rows)
    args = (dev(x, torch.bfloat16), dev(weight, torch.bfloat16), dev(table, torch.bfloat16), dev(ids, torch.int32))
    got = ops.linear_gelu_table(*args, features + 3)
    two = ops.gated_table_rows(ops.linear(args[0], args[1]), args[2], args[3], features + 3)
    assert torch.equal(got, two)
    gate = tn.bf16_round((x.astype(np.float64) @ weight.astype(np.float64).T).astype(np.float32)).astype(np.float64)
    want = pn.gelu_tanh(gate) * table[ids, features + 3 : 2 * features + 3]
    assert np.abs(got.float().cpu().numpy() - want).max() < tolerance("bfloat16", max(1.0, np.abs(want).max()))


@pytest.mark.parametrize("rows, width, k", [(1, 24, 64), (8, 70, 256), (16, 256, 512), (5, 16, 32)])
def test_stacked_product_with_one_step_of_the_recurrence_in_its_last_step(rows, width, k):
    """Single tokens of several requests: the fused kernel leaves the outputs and the state rows that
    the product followed by the recurrence kernel leaves, bit for bit; rows of other slots stay."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(rows * width)
    slots_n = 20
    x = dev(tn.bf16_round(rng.standard_normal((rows, k)).astype(np.float32)), torch.bfloat16)
    weight = dev(tn.bf16_round((2.0 * rng.standard_normal((3 * width, k)) / np.sqrt(k)).astype(np.float32)), torch.bfloat16)
    bz, bx = dev(rng.standard_normal(width).astype(np.float32)), dev(rng.standard_normal(width).astype(np.float32))
    start = rng.standard_normal((slots_n + 1, width + 6)).astype(np.float32)
    owners = rng.permutation(slots_n)[:rows].astype(np.int32)
    if rows > 1:
        owners[1] = -1  # a padding row of a recorded step: nobody's state row
    cu = dev(np.arange(rows + 1), torch.int32)
    fused_buffer, plain_buffer = dev(start), dev(start)
    fused_state, plain_state = fused_buffer[:, 2 : 2 + width], plain_buffer[:, 2 : 2 + width]
    fused = ops.linear_gru(x, weight, bz, bx, fused_state, dev(owners, torch.int32))
    plain = ops.gated_scan(ops.linear(x, weight), bz, bx, plain_state, cu, dev(owners, torch.int32), 1)
    assert torch.equal(fused, plain) and torch.equal(fused_buffer, plain_buffer)
    untouched = sorted(set(range(slots_n)) - set(int(o) for o in owners))
    assert np.array_equal(fused_buffer.cpu().numpy()[untouched], start[untouched])


# ---------------------------------------------------------------------------------------------
# whole models under schedules
# ---------------------------------------------------------------------------------------------

LENGTHS = {"P": (83, 1, 40, 23, 61, 97), "Q": (45, 2, 30, 19, 52), "R": (70, 37, 90, 5), "S": (33, 20, 1, 48, 27)}


def requests_of(name, cfg):
    return {f"{name}{i}": tn.random_tokens(cfg, n, seed=100 * len(name) + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(tn.CONFIGS))
@pytest.mark.parametrize("family", ["whole", "decode", "portions", "mixed"])
def test_logits_do_not_depend_on_the_schedule(folders, name, dtype, family):
    """Whole prompts; a prompt and then its last tokens one by one, past every window; portions
    down to two tokens; up to four live requests of unequal length in one batch, in a pool so small
    that pages and state slots are used again.  Each request is held against itself alone."""
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


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_and_pages_used_again_start_clean(folders, dtype):
    """One seat, pages for one request: the second request gets the first one's slot and pages."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["P"]
    first, second = tn.random_tokens(cfg, 30, seed=1), tn.random_tokens(cfg, 26, seed=2)
    runner = runner_for(folder, dtype, block, pages=2, seats=1)
    runner.step([StepEntry("a", first, [])])
    slot = runner.cache.state_slot("a")
    runner.free_request("a")
    got = runner.step([StepEntry("b", second[:9], list(range(9)))]).cpu().numpy()
    assert runner.cache.state_slot("b") == slot
    got = np.concatenate([got, runner.step([StepEntry("b", second[9:], list(range(17)))]).cpu().numpy()])
    ru.assert_close(got, oracle("P", cfg, weights, second), dtype, "second owner of a slot")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_recorded_steps(folders, dtype):
    """Two requests decoded side by side for 150 steps after short prompts (windows of 24 and 7 pass
    many times, pages are given back behind them); the single-token steps are replayed graphs."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["P"]
    requests = {"x": tn.random_tokens(cfg, 153, seed=31), "y": tn.random_tokens(cfg, 157, seed=32)}
    runner = runner_for(folder, dtype, block, pages=8, seats=2)
    got = {rid: [] for rid in requests}
    both = runner.step([StepEntry("x", requests["x"][:3], [0, 1, 2]), StepEntry("y", requests["y"][:7], list(range(7)))]).cpu().numpy()
    got["x"].append(both[:3])
    got["y"].append(both[3:])
    for k in range(150):
        logits = runner.step([StepEntry("x", [requests["x"][3 + k]], [0]), StepEntry("y", [requests["y"][7 + k]], [0])]).cpu().numpy()
        got["x"].append(logits[:1])
        got["y"].append(logits[1:])
    assert runner.decode_graphs is not None and runner.decode_graphs.replays == 150
    for rid, tokens in requests.items():
        ru.assert_close(np.concatenate(got[rid]), oracle("P", cfg, weights, tokens), dtype, f"long decoding {rid}")
    # the windows have passed: only the pages that the last queries can see are still held
    assert runner.num_free_blocks() >= 8 - 2 * 3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window, block", [(16, 16), (17, 16), (33, 8), (150, 16)])
def test_keys_just_inside_and_just_outside_a_window_in_prompts_and_in_decoding(tmp_path, dtype, window, block):
    """One attention layer with peaked scores between two recurrent layers; windows that end on a
    page border, one key past it, and many pages long.  The engine must agree with the plain
    model of this window and be far from the plain models whose window is one key longer or shorter."""
    from mini_infer_amd.engine import StepEntry

    def cfg_with(size):
        return tn.config(64, 64, [tn.mingru(32), tn.attention(2, 1, 32, size, 0.9, ff=48), tn.mingru(40)],
                         scale=2.0, eps=1e-6, side=4)

    cfg = cfg_with(window)
    weights = tn.make_weights(cfg, seed=window)
    tokens = tn.random_tokens(cfg, window + 60, seed=window + 1)
    folder = tn.write_model_dir(tmp_path / "m", cfg, weights)
    right = ru.Oracle(pn.logits(cfg, weights, tokens), pn.logits(cfg, weights, tokens, store=pn.bf16_round))
    wrong = [pn.logits(cfg_with(window + d), weights, tokens) for d in (-1, 1)]
    head = window + 20  # the prompt itself passes the window; 40 more tokens one by one
    runner = runner_for(folder, dtype, block, pages=-(-len(tokens) // block), seats=1)
    rows = [runner.step([StepEntry("w", tokens[:head], list(range(head)))]).cpu().numpy()]
    rows += [runner.step([StepEntry("w", [t], [0])]).cpu().numpy() for t in tokens[head:]]
    got = np.concatenate(rows)
    ru.assert_close(got, right, dtype, f"window {window}")
    past = slice(window, None)  # from here on a window one key off sees another set of keys
    error = np.abs(got[past] - right.exact[past]).max(axis=1)
    for other in wrong:
        apart = np.abs(other[past] - right.exact[past]).max(axis=1)
        if dtype == "float32":
            assert np.median(apart) > 20 * np.median(error) and (apart > error).mean() > 0.95
        elif window <= 33:  # (one key in 150 moves the logits by less than bfloat16 does)
            assert apart.max() > 3 * error.max()


def test_a_lost_state_or_a_gain_left_out_would_show(folders, dtype="float32"):
    """The tests above can only be trusted if the tiny weights make each mechanism matter: the plain
    model with one mechanism switched off must differ from the full one by far more than the
    engine does."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["P"]
    tokens = tn.random_tokens(cfg, 50, seed=77)
    full = oracle("P", cfg, weights, tokens)
    runner = runner_for(folder, dtype, block, pages=4, seats=1)
    got = runner.step([StepEntry("a", tokens, list(range(50)))]).cpu().numpy()
    error = np.abs(got - full.exact).max()

    def without(change):
        other = {k: v.copy() for k, v in weights.items()}
        change(other)
        return np.abs(pn.logits(cfg, other, tokens) - full.exact).max()

    switched_off = {
        "layer scale": lambda w: w.update({"l1.ls1": np.ones_like(w["l1.ls1"])}),
        "one-number gain": lambda w: w.update({"l2.norm2": np.float32(1.0)}),
        "key norm weight": lambda w: w.update({"l0.mix.k.norm": np.ones_like(w["l0.mix.k.norm"])}),
        "recurrence bias": lambda w: w.update({"l1.mix.z.b": np.zeros_like(w["l1.mix.z.b"])}),
        "side input": lambda w: w.update({"side.embed": np.zeros_like(w["side.embed"])}),
        "activation offset": lambda w: w.update({"l0.mlp.act": w["l0.mlp.act"] * np.array([1, 1, 1, 0], dtype=np.float32)}),
        "final gain": lambda w: w.update({"final.norm": np.float32(1.0)}),
    }
    for what, change in switched_off.items():
        assert without(change) > max(0.02, 1000 * error), what
    cut = np.abs(np.concatenate([pn.logits(cfg, weights, tokens[:25]), pn.logits(cfg, weights, tokens[25:])]) - full.exact).max()
    assert cut > max(0.02, 1000 * error)  # a state or a cache lost between portions


# ---------------------------------------------------------------------------------------------
# through the framework's own entry points
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["P", "S"])
def test_greedy_generation_through_llm_and_the_scheduler(folders, name):
    """Five prompts for two seats, prompts cut into portions of 8 under a 20-token budget: every
    generated token is the plain model's greedy choice."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = folders[name]
    lengths, new_tokens = (5, 19, 33, 2, 11), 9
    prompts = [tn.random_tokens(cfg, n, seed=300 + n) for n in lengths]
    llm = LLM(folder, dtype="float32", num_blocks=12, block_size=block, max_concurrent=2, max_num_batched_tokens=20, chunk_size=8)
    results = llm.generate(prompts, max_tokens=new_tokens)
    for prompt, result in zip(prompts, results):
        sequence = list(prompt)
        for _ in range(new_tokens):
            sequence.append(pn.greedy(pn.logits(cfg, weights, sequence)[-1]))
        assert result.tokens == sequence[len(prompt):] and result.finish_reason == "length"
    assert llm.runner.cache.states.num_free == 2
    llm.runner.cache.check()


def test_the_replay_program_runs_a_trace_of_this_design(folders, tmp_path):
    from mini_infer_amd.engine import replay, trace

    cfg, block, weights, folder = folders["Q"]
    requests = {f"t{i}": tn.random_tokens(cfg, n, seed=i) for i, n in enumerate((70, 41, 9, 33, 58))}
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
            want = oracle("Q", cfg, weights, requests[rid])[slice(fed[rid], fed[rid] + n)]
            ru.assert_close(got[at : at + n], want, "float32", f"trace step {number} {rid}")
            fed[rid] += n
            at += n
