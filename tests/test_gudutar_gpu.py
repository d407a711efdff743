"""Gudutar in the engine against the plain implementation under tests/plain/: each mechanism alone, whole prompts,
token-by-token decoding, portions down to two tokens, unequal requests in one batch with pages and state slots used
again, the edges of the attention window and state carried over hundreds of tokens (with inputs made so that a fault
shows), the first tokens of a sequence, sizes of several kinds, and greedy generation through ``LLMEngine``."""

import os

import numpy as np
import pytest
import torch

from tests import helpers
from tests.gudutar_configs import ALONE, GUDU_A, GUDU_B, GUDU_C
from tests.helpers import TraceBuilder
from tests.plain import gudutar_plain as plain

pytestmark = pytest.mark.gpu

CONFIGS = {"A": GUDU_A, "B": GUDU_B, "C": GUDU_C, **ALONE}
TOL = {"float32": 3e-5, "bfloat16": 6e-2}


def write_folder(path, cfg, seed, stored, edit=None):
    """A model folder with random weights (norm weights near one, everything else normal with the width's scale);
    ``edit(tensors)`` may change them before they are stored."""
    from safetensors.torch import load_file, save_file
    from paged_llm_amd.weights import write_random_model
    folder = write_random_model(str(path), cfg, seed=seed, dtype=stored, std=cfg["width"] ** -0.5, norm_jitter=True)
    if edit is not None:
        file = os.path.join(folder, "model.safetensors")
        tensors = load_file(file)
        edit(tensors)
        save_file({k: v.contiguous() for k, v in tensors.items()}, file)
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, stored):
        if (name, stored) not in made:
            made[name, stored] = write_folder(tmp_path_factory.mktemp(f"gudutar_{name}_{stored}"), CONFIGS[name],
                                              seed=11 + len(name), stored=stored)
        return made[name, stored]
    return get


_plain_cache: dict = {}


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = plain.forward(plain.read_config(folder), plain.load_weights(folder), list(tokens)).numpy()
    return _plain_cache[key]


def session_for(folder, dtype, max_tokens, **kw):
    from paged_llm_amd.engine.replay import ReplaySession
    return ReplaySession(folder, dtype, max_tokens, None, **kw)


_noise_cache: dict = {}


def rounding_scale(folder, tokens):
    """Per position: how far the plain logits move (root mean square over four draws of ``helpers.worst``) when every
    product's rows and result carry the relative error of bfloat16 rounding.  Some positions of these small random models
    are far more sensitive than others (the first token of a retention layer is (q . k) v divided by its root mean
    square, which is the sign of q . k: where that product is nearly zero, rounding decides the sign; a softmax between
    two near-equal scores), so a bfloat16 result is judged against its own position's scale."""
    key = (folder, tuple(tokens))
    if key not in _noise_cache:
        exact = plain_logits(folder, tokens)
        cfg, weights = plain.read_config(folder), plain.load_weights(folder)
        sq = np.zeros(len(tokens))
        for seed in range(4):
            with plain.rounding_noise(seed):
                moved = plain.forward(cfg, weights, list(tokens)).numpy()
            sq += (np.abs(moved - exact).max(axis=1) / np.abs(exact).max(axis=1)) ** 2
        _noise_cache[key] = np.sqrt(sq / 4)
    return _noise_cache[key]


_exact_cache: dict = {}


def float32_scale(folder, tokens):
    """Per position: how far the plain implementation in float32 is from itself in float64.  Where a head's output is a
    sum that nearly cancels and is then divided by its root mean square, float32 rounding alone moves a row by far more
    than elsewhere, and another order of the same additions (chunks instead of token by token) moves it as much."""
    key = (folder, tuple(tokens))
    if key not in _exact_cache:
        exact = plain.forward(plain.read_config(folder), plain.load_weights(folder), list(tokens), dtype=torch.float64).numpy()
        _exact_cache[key] = np.abs(plain_logits(folder, tokens) - exact).max(axis=1) / np.abs(exact).max(axis=1)
    return _exact_cache[key]


def bound_at(folder, tokens, pos, dtype, floor32=None):
    """What a row may differ by: in float32 3e-5, or 5 times the plain implementation's own float32 error at that position
    if that is more; in bfloat16 4 times the position's rounding scale, at least 3e-2."""
    if dtype == "float32":
        return max(floor32 or TOL[dtype], 5.0 * float(float32_scale(folder, tokens)[pos]))
    return max(3e-2, 4.0 * float(rounding_scale(folder, tokens)[pos]))


def check(got: dict, folder, reqs: dict, dtype, floor32=None, narrow=False):
    """Every row within its bound in float32 (``floor32``: another least bound than 3e-5); in bfloat16 no row beyond twice its bound and at most one in fifty beyond
    it, and the median error below 2.5e-2."""
    want = {rid: plain_logits(folder, toks) for rid, toks in reqs.items()}
    ratios, errs = {}, []
    for (rid, pos), row in got.items():
        err = helpers.worst(row, want[rid][pos])
        errs.append(err)
        ratios[rid, pos] = err / bound_at(folder, reqs[rid], pos, dtype, floor32)
    worst_at = max(ratios, key=ratios.get)
    said = f"{worst_at}: {ratios[worst_at]:.3g} of its bound (median error {np.median(errs):.3g})"
    if dtype == "float32":
        assert ratios[worst_at] <= 1.0, said
    else:
        over = sum(1 for r in ratios.values() if r > 1.0)
        # (narrow: models a few dozen channels wide, whose rows move more under rounding and whose few draws of the
        #  yardstick say less: twice the allowances; a fault in a kernel moves most rows by their whole size)
        most, middle = (4.0, 5e-2) if narrow else (2.0, 2.5e-2)
        assert ratios[worst_at] <= most and over <= max(1, len(ratios) // 50) and np.median(errs) <= middle, f"{said}, {over} rows over"


def rounded(n):
    return -(-n // 64) * 64


def whole(reqs):
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        trace.step([(rid, toks, "all")], end=[rid])
    return trace


def stored_as(dtype):
    return "float32" if dtype == "float32" else "bfloat16"


# --------------------------------------------------------------------------- each mechanism alone, and whole models
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts(folders, name, dtype):
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    reqs = {"p1": helpers.random_tokens(1, vocab, 1), "p5": helpers.random_tokens(5, vocab, 2), "p70": helpers.random_tokens(70, vocab, 3)}
    got = helpers.replay_in_process(session_for(folder, dtype, 128), whole(reqs))
    assert len(got) == 76
    check(got, folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "mamba2", "retention", "latent_attention"])
def test_prompt_then_token_by_token(folders, name, dtype):
    """A prompt in one step and then single tokens: cache, state slots and the window behind decoded tokens."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(75, CONFIGS[name]["vocab"], 7)
    trace = TraceBuilder().step([("r", toks[:13], "all")])
    for i in range(13, 75):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 74 else [])
    session = session_for(folder, dtype, 128)
    check(helpers.replay_in_process(session, trace), folder, {"r": toks}, dtype)
    assert any(key[0] != "prompt" for key in session.runner._graphs), "single-token steps are replayed from graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_token_by_token_from_the_first(folders, dtype):
    """No prompt step at all: the first tokens meet the convolution's zeros and an empty state."""
    folder = folders("A", stored_as(dtype))
    toks = helpers.random_tokens(9, GUDU_A["vocab"], 8)
    trace = TraceBuilder()
    for i in range(9):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 8 else [])
    check(helpers.replay_in_process(session_for(folder, dtype, 64), trace), folder, {"r": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16, 1, 17, 2, 31], [64, 5]])
def test_portions(folders, name, dtype, sizes):
    """Prompts cut into portions of several sizes, down to two tokens (shorter than the convolution's reach), cut in the
    middle of pages and of the window."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(97, CONFIGS[name]["vocab"], 9)
    trace, at, k = TraceBuilder(), 0, 0
    while at < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - at)
        trace.step([("r", toks[at:at + n], "all")], end=["r"] if at + n == len(toks) else [])
        at, k = at + n, k + 1
    check(helpers.replay_in_process(session_for(folder, dtype, 128), trace), folder, {"r": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_logits_do_not_depend_on_the_cut(folders, name, dtype):
    """The same request whole, in portions and token by token: equal within rounding of the compute type, and far
    inside the bound against the plain implementation in float32."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(60, CONFIGS[name]["vocab"], 10)
    a = helpers.replay_in_process(session_for(folder, dtype, 64), whole({"r": toks}))
    trace = TraceBuilder().step([("r", toks[:31], "all")]).step([("r", toks[31:33], "all")])
    for i in range(33, 60):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 59 else [])
    b = helpers.replay_in_process(session_for(folder, dtype, 64), trace)
    if dtype == "float32":
        assert max(helpers.worst(b[k], a[k]) for k in a) <= 1e-5
    else:
        assert max(helpers.worst(b[k], a[k]) / bound_at(folder, toks, k[1], dtype) for k in a) <= 2.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_long_portions_run_in_chunks(folders, name, dtype):
    """Portions of 128 tokens and more take the recurrences' chunked form (a chunk's own state from zero, the states
    carried from chunk to chunk, outputs from each chunk's starting state): lengths at, just past and between the
    chunks' borders, a second long portion that starts from a carried state, and short and single-token sequences beside
    a long one in the same step."""
    from paged_llm_amd.csrc import ops
    assert ops.recurrence_chunk(128, 300) == 16 and ops.recurrence_chunk(127, 300) == 0 and ops.recurrence_chunk(2048, 2048) == 64
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    reqs = {"long": helpers.random_tokens(449, vocab, 20), "side": helpers.random_tokens(150, vocab, 21),
            "short": helpers.random_tokens(30, vocab, 22)}
    trace = TraceBuilder()
    trace.step([("short", reqs["short"][:9], "all")])
    trace.step([("short", reqs["short"][9:10], "all"), ("long", reqs["long"][:129], "all")])           # 129 = two chunks and one token
    trace.step([("short", reqs["short"][10:11], "all"), ("side", reqs["side"][:5], "all"), ("long", reqs["long"][129:320], "all")])
    trace.step([("side", reqs["side"][5:133], "all"), ("long", reqs["long"][320:448], "all")])         # two portions of 128
    trace.step([("long", reqs["long"][448:], "all"), ("side", reqs["side"][133:], "all"), ("short", reqs["short"][11:], "all")],
               end=["long", "side", "short"])
    got = helpers.replay_in_process(session_for(folder, dtype, 64 * 8 + 192 + 64), trace)
    assert len(got) == 449 + 150 + 30
    # (the chunks add the same terms into the state in another order than the plain implementation's token-by-token loop,
    #  whose own float32 roundings the token-by-token kernel repeats one for one: where a head's output nearly cancels
    #  the two orders differ by 1e-4; a fault in the chunks' bookkeeping would show as a difference of order one)
    check(got, folder, reqs, dtype, floor32=3e-4)


# --------------------------------------------------------------------------- batches, pages and slots used again
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    from tests.test_replay_gpu import mixed_trace
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    lengths = [33, 1, 90, 17, 64, 5, 48, 2, 71]
    reqs = {f"q{i}": helpers.random_tokens(n, vocab, 40 + i) for i, n in enumerate(lengths)}
    trace, peak = mixed_trace(reqs, max_live=3, seed=3)
    session = session_for(folder, dtype, peak, max_requests=3)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == sum(lengths)
    check(got, folder, reqs, dtype)
    session.manager.check_invariants()
    assert session.manager.slots.num_free == session.manager.slots.num_slots == 3
    assert all(session.manager.num_free_pages(g) == session.manager.num_pages(g) for g in session.manager.groups)
    kinds = {"prompt" if key[0] == "prompt" else "decode" for key in session.runner._graphs}
    assert kinds == {"prompt", "decode"}, "steps of both kinds were replayed from graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_that_held_another_request_starts_from_zero(folders, dtype):
    """One state slot, one page pool of one request: the second request gets the slot and pages the first one left full."""
    folder = folders("A", stored_as(dtype))
    reqs = {"first": helpers.random_tokens(50, GUDU_A["vocab"], 60), "second": helpers.random_tokens(44, GUDU_A["vocab"], 61)}
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        trace.step([(rid, toks[:20], "all")])
        trace.step([(rid, toks[20:22], "all")])
        for i in range(22, len(toks)):
            trace.step([(rid, toks[i:i + 1], "all")], end=[rid] if i == len(toks) - 1 else [])
    session = session_for(folder, dtype, 64, max_requests=1)
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


# --------------------------------------------------------------------------- where random weights would hide a fault
def _boost(token, factor):
    def edit(tensors):
        tensors["embed"][token] = (tensors["embed"][token].float() * factor).to(tensors["embed"].dtype)
    return edit


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edges_in_prompts_and_in_decoding(tmp_path, dtype):
    """A token whose embedding is several times larger than the others' stands at one place; its key then dominates the
    softmax of the queries that see it.  The positions at which it is last seen and first hidden (window - 1 and window
    tokens later) are compared with the plain implementation, whole and decoded; the plain implementation with a window
    one shorter or longer differs by far more than the bound there, so a window that is one token off would show."""
    cfg = ALONE["latent_attention"]
    window, special, at = cfg["layers"][0]["mixer"]["mask"]["size"], 7, 30
    folder = write_folder(tmp_path, cfg, seed=5, stored=stored_as(dtype), edit=_boost(special, 6.0))
    toks = [t if t != special else special + 1 for t in helpers.random_tokens(64, cfg["vocab"], 12)]
    toks[at] = special
    edge_in, edge_out = at + window - 1, at + window
    want = plain_logits(folder, toks)
    for off_by in (-1, 1):                                 # the plain implementation with another window: the test can tell
        other = plain.read_config(folder)
        other["layers"][0]["mixer"]["mask"]["size"] = window + off_by
        moved = plain.forward(other, plain.load_weights(folder), toks).numpy()
        pos = edge_in if off_by < 0 else edge_out
        assert helpers.worst(moved[pos], want[pos]) > 4 * bound_at(folder, toks, pos, dtype), "the special token does not show at the window's edge"
    for cut in (64, edge_in - 3, at + 1):                   # whole; the edge among decoded tokens; all of the window decoded
        trace = TraceBuilder().step([("r", toks[:cut], "all")], end=["r"] if cut == 64 else [])
        for i in range(cut, 64):
            trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 63 else [])
        got = helpers.replay_in_process(session_for(folder, dtype, 64), trace)
        for pos in (edge_in - 1, edge_in, edge_out, edge_out + 1):
            err = helpers.worst(got["r", pos], want[pos])
            assert err <= 2.0 * bound_at(folder, toks, pos, dtype), f"cut {cut}, position {pos}: {err:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["retention", "mamba2"])
def test_a_token_far_back_still_shows(tmp_path, name, dtype):
    """The recurrent state carries one early, large token over hundreds of tokens, through portions, page borders and
    decoded tokens; the plain implementation without that token differs far beyond the bound at the end, so a state
    that was lost or reset on the way would show."""
    cfg = ALONE[name]
    if name == "retention":                                 # decays close to one, or nothing is left after 300 tokens
        cfg = {**cfg, "layers": [{**cfg["layers"][0], "mixer": {**cfg["layers"][0]["mixer"], "decay": [0.999, 0.9999]}}]}
    special = 3

    def edit(tensors):
        _boost(special, 8.0)(tensors)
        if name == "mamba2":                                # slow decay: exp(A_log) small, so that the state keeps the token
            tensors["l0.mix.A_log"] = torch.full_like(tensors["l0.mix.A_log"], -6.0)
    folder = write_folder(tmp_path, cfg, seed=6, stored=stored_as(dtype), edit=edit)
    toks = [t if t != special else special + 1 for t in helpers.random_tokens(330, cfg["vocab"], 13)]
    toks[2] = special
    want = plain_logits(folder, toks)
    without = plain.forward(plain.read_config(folder), plain.load_weights(folder), toks[:2] + [special + 1] + toks[3:]).numpy()
    # (against the float32 bound: in bfloat16 the same kernels run, instantiated for the other storage type)
    assert helpers.worst(without[-1], want[-1]) > 10 * TOL["float32"], "the early token does not show at the end"
    trace, at = TraceBuilder(), 0
    for n in (17, 2, 64, 100, 3, 96):
        trace.step([("r", toks[at:at + n], "last")])
        at += n
    for i in range(at, 330):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 329 else [])
    check(helpers.replay_in_process(session_for(folder, dtype, 384), trace), folder, {"r": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    folder = folders("B", stored_as(dtype))
    toks = helpers.random_tokens(300, GUDU_B["vocab"], 14)
    trace = TraceBuilder().step([("r", toks[:4], "all")])
    for i in range(4, 300):
        trace.step([("r", toks[i:i + 1], "all" if i % 7 == 0 or i > 280 else [])], end=["r"] if i == 299 else [])
    check(helpers.replay_in_process(session_for(folder, dtype, 320), trace), folder, {"r": toks}, dtype)


# --------------------------------------------------------------------------- the entry point and its scheduler
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(folders, name):
    """``LLMEngine.generate`` with portions of 16 tokens, three requests at a time for five prompts (state slots and pages
    are used again): in float32 the tokens are the plain implementation's greedy choice, in bfloat16 every row the engine
    sampled from is within the bound of the plain logits along its own tokens."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    vocab = CONFIGS[name]["vocab"]
    prompts = [helpers.random_tokens(n, vocab, 70 + n) for n in (3, 41, 18, 1, 29)]
    for dtype in ("float32", "bfloat16"):
        folder = folders(name, stored_as(dtype))
        engine = LLMEngine(folder, EngineConfig(dtype=dtype, num_gpu_blocks=24, block_size=16, max_num_batched_tokens=16,
                                                max_num_seqs=3, max_model_len=128))
        rows = {}

        def keep(requests, logits):
            for r, row in zip(requests, logits.float().cpu()):
                rows[r.id, len(r.tokens) - 1] = row.numpy()
        engine.on_logits = keep
        outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
        assert engine.cache_manager.slots.num_free == 3
        for p, o in zip(prompts, outs):
            assert len(o.token_ids) == 12
            want = plain_logits(folder, p + o.token_ids)
            for i, token in enumerate(o.token_ids):
                pos = len(p) + i - 1
                err = helpers.worst(rows[o.seq_id, pos], want[pos])
                assert err <= 2.0 * bound_at(folder, p + o.token_ids, pos, dtype) and int(rows[o.seq_id, pos].argmax()) == token, (dtype, pos, err)
                if dtype == "float32":
                    top2 = np.sort(want[pos])[-2:]
                    if top2[1] - top2[0] > 1e-3 * np.abs(want[pos]).max():
                        assert token == int(want[pos].argmax()), (pos, token)


def test_the_command_line_generates(folders, capsys):
    import importlib.util
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("generate_example", os.path.join(root, "examples", "generate.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    code = mod.main(["--model", folders("A", "bfloat16"), "--prompt-ids", "5,6,7", "--prompt-ids", "9", "--max-tokens", "6",
                     "--num-gpu-blocks", "16", "--max-model-len", "64", "--ignore-eos"])
    out = capsys.readouterr().out
    assert code == 0 and "decode_tokens=" in out and out.count("--- [") == 2


# --------------------------------------------------------------------------- the replay program, and sizes drawn at random
def test_the_replay_program(folders, tmp_path):
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders("A", "float32")
    toks = {"a": helpers.random_tokens(70, GUDU_A["vocab"], 90), "b": helpers.random_tokens(45, GUDU_A["vocab"], 91)}
    trace = TraceBuilder()
    trace.step([("a", toks["a"][:50], [0, 49])])
    trace.step([("a", toks["a"][50:52], "all"), ("b", toks["b"][:30], [])])
    trace.step([("b", toks["b"][30:], "last"), ("a", toks["a"][52:53], "all")], end=["b"])
    trace.step([("a", toks["a"][53:], "all")], end=["a"])
    out_dir = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out_dir),
                           "--max-tokens", "192"], input=trace.jsonl(), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3"]
    got = helpers.read_replay_output(str(out_dir), trace, GUDU_A["vocab"])
    assert len(got) == 2 + 2 + 1 + 1 + 17
    check(got, folder, toks, "float32")


def random_configuration(seed: int) -> dict:
    """A Gudutar configuration with every size drawn at random (small ones, ones and odd ones included) and the three
    mixers in a random order, some layers with borrowed weights."""
    from tests.gudutar_configs import _latent, _layer, _mamba, _retention, model
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    made = {}

    def mixer(kind):
        if kind == "mamba2":
            groups = pick(1, 2, 3)
            heads = groups * pick(1, 2, 3)
            vdim = pick(1, 2, 5, 8, 20, 33, 70)
            parts = pick(*[d for d in (1, 2, 3, 4, 5) if (heads * vdim) % d == 0])
            return _mamba(heads=heads, vdim=vdim, state=pick(1, 3, 16, 40, 64, 65, 130), groups=groups, conv=pick(1, 2, 4, 5), norm_groups=parts)
        if kind == "retention":
            heads, dim = pick(1, 2, 5), pick(2, 6, 16, 34, 70)
            return _retention(heads=heads, dim=dim, vdim=pick(1, 3, 16, 40, 66), rot_dims=pick(*[d for d in (2, 4, 6, 16, 34) if d <= dim]),
                              base=pick(10.0, 1e4, 1e6), decay=[float(rng.uniform(0.3, 0.9999)) for _ in range(heads)])
        rot = pick(2, 4, 8, 18)
        return _latent(heads=pick(1, 2, 5, 8), dim=pick(1, 4, 16, 30), rot_dim=rot, vdim=pick(1, 4, 24, 50), kv_rank=pick(3, 16, 40, 100, 260),
                       window=pick(0, 1, 2, 7, 16, 33, 100), base=pick(10.0, 1e4), scale=float(rng.uniform(0.05, 0.5)))

    layers = []
    for i in range(int(rng.integers(2, 6))):
        kind = pick("mamba2", "retention", "latent_attention")
        if kind in made and rng.random() < 0.3:
            layers.append(_layer(kind, None, weights_of=made[kind]))
        else:
            made.setdefault(kind, i)
            layers.append(_layer(kind, mixer(kind), ff=pick(None, None, 10, 36, 65)))
    return model(pick(16, 30, 48, 66, 100), pick(40, 97, 300), layers, eps=pick(1e-6, 1e-5, 1e-3), scale=float(rng.uniform(0.5, 12.0)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    """Whatever the sizes, the engine computes what the plain implementation computes, whole, in portions and token by
    token, two requests side by side."""
    cfg = random_configuration(seed)
    folder = write_folder(tmp_path, cfg, seed=100 + seed, stored=stored_as(dtype))
    reqs = {"a": helpers.random_tokens(150, cfg["vocab"], 200 + seed), "b": helpers.random_tokens(37, cfg["vocab"], 300 + seed)}
    trace = TraceBuilder()
    trace.step([("a", reqs["a"][:130], "all")])                                       # a long portion: the chunked recurrences
    trace.step([("a", reqs["a"][130:132], "all"), ("b", reqs["b"][:20], "all")])
    for i in range(17):
        trace.step([("a", reqs["a"][132 + i:133 + i], "all"), ("b", reqs["b"][20 + i:21 + i], "all")], end=["b"] if i == 16 else [])
    trace.step([("a", reqs["a"][149:], "all")], end=["a"])
    got = helpers.replay_in_process(session_for(folder, dtype, 256), trace)
    assert len(got) == 150 + 37
    check(got, folder, reqs, dtype, floor32=3e-4, narrow=True)


def test_preempted_requests_start_again_from_an_empty_state(folders):
    """A page pool too small for three requests at once: the scheduler preempts the request admitted last (pages and state
    slot given back, its tokens kept) and computes it again later as a longer prompt, from position 0 and so from a zero
    state in whatever slot it gets.  Float32: the tokens are the plain implementation's greedy choice all the same."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    folder = folders("B", "float32")
    vocab = GUDU_B["vocab"]
    prompts = [helpers.random_tokens(n, vocab, 400 + n) for n in (30, 22, 27)]
    engine = LLMEngine(folder, EngineConfig(dtype="float32", num_gpu_blocks=10, block_size=16, max_num_batched_tokens=32,
                                            max_num_seqs=3, max_model_len=128))
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True))
    assert engine.stats.num_preemptions > 0 and sum(o.num_preemptions for o in outs) > 0
    assert engine.cache_manager.slots.num_free == 3
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 40
        want = plain_logits(folder, p + o.token_ids)
        for i, token in enumerate(o.token_ids):
            row = want[len(p) + i - 1]
            top2 = np.sort(row)[-2:]
            if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
                assert token == int(row.argmax()), (len(p), i)
