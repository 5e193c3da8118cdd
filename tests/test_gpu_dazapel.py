"""The Dazapel decoder on the GPU against the plain implementation in ``plain_dazapel.py``: each
mechanism alone, whole prompts, decoding, portions, mixed batches, pages and slots used again, peaked
attention at the edges of windows and among the kept first tokens, sizes that are 1, equal or odd, and
greedy generation through ``LLM``."""

import copy

import pytest
import torch

import dazapel_util as du
import plain_dazapel as plain
from replay_util import mixed_trace, portion_trace, random_tokens, round64, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu

F64 = torch.float64


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("mixed", du.MIXED, 21), ("sharp", du.SHARP, 22), ("ones", du.ONES, 23), ("odd", du.ODD, 24)):
        out[name] = du.write_model(str(tmp_path_factory.mktemp(name)), cfg, seed)
    return out


def _oracle(folder, tokens, store=None, cfg_edit=None):
    cfg, tensors = plain.dazapel_read(folder, F64)
    if cfg_edit is not None:
        cfg_edit(cfg)
    return plain.dazapel_forward(cfg, tensors, tokens, store or plain._keep).to(torch.float32)


def _rel(got, want):
    """Per row: RMS of the difference (mean taken off) over the RMS of the wanted row."""
    d = (got - want).double()
    d = d - d.mean(dim=1, keepdim=True)
    return (d.pow(2).mean(dim=1).sqrt() / want.double().pow(2).mean(dim=1).sqrt()).max().item()


def _rel_rows(got, want):
    d = (got - want).double()
    d = d - d.mean(dim=1, keepdim=True)
    return d.pow(2).mean(dim=1).sqrt() / want.double().pow(2).mean(dim=1).sqrt()


def _like_rounding(errors, rounding):
    """``errors``: per-row distances of the engine's bfloat16 logits from exact arithmetic; ``rounding``:
    the same for the plain model with its stored activations rounded to bfloat16.  Rounding moves single
    rows far (a router's choice between two experts whose scores all but tie falls the other way, a peaked
    softmax picks the neighbour), in the plain model as in the engine, so the two are compared as
    distributions: the middle row and the row that nine in ten stay below."""
    return (errors.median() < 2 * rounding.median() + 1e-3
            and errors.quantile(0.9) < 3 * rounding.quantile(0.9) + 1e-3)


def _replayer(folder, dtype, max_tokens, max_live=4):
    from qwen25vl_lite_amd.engine.replay import Replayer
    return Replayer(folder, dtype, max_tokens, 16, max_live)


def _rows(got, rid, n):
    return torch.stack([got[(rid, p)] for p in range(n)])


# ---------------------------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------------------------
def _one_layer(tmp_path, lay, dtype=torch.float32, seed=0, width=56):
    from qwen25vl_lite_amd.config import EngineConfig, load_config
    from qwen25vl_lite_amd.engine import ModelRunner
    from qwen25vl_lite_amd.models import build_model
    from qwen25vl_lite_amd.weights import load_weights
    cfg = du.config(width, 50, [lay], eps=1e-4)
    d = du.write_model(str(tmp_path / "one"), cfg, seed)
    model = build_model(load_config(d), dtype, "cuda:0")
    load_weights(d, model)
    ecfg = EngineConfig(num_blocks=32, block_size=16, max_num_seqs=3, max_num_batched_tokens=256, max_model_len=256,
                        enable_prefix_cache=False, dtype=dtype)
    _, tensors = plain.dazapel_read(d, F64)
    return ModelRunner(model, ecfg), model.blocks[0], tensors


def _step_for(runner, rid, n, start=0):
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.engine.batch import build_step
    if start == 0:
        runner.admit(rid)
    e = StepEntry(rid, [0] * n, start)
    runner.cache.reserve(rid, start + n)
    return build_step([e], runner.cache, 1, runner.dtype, runner.device)


@pytest.mark.parametrize("mask", [None, (7, 3), (70, 0), (3, 40)])
def test_attention_alone_whole_and_in_two_steps(mask, tmp_path):
    m = du.attention(4, 2, 20, 12, 12, base=300.0, scaling=du.RAMP, scale=1.4, mask=mask)
    runner, block, t = _one_layer(tmp_path, du.layer(m))
    torch.manual_seed(5)
    n = 90
    x = torch.randn(n, 56, dtype=F64)
    want = plain.attention_mixer(x, t, "l0.mix.", m, 1e-4)
    step = _step_for(runner, "a", n)
    got = block.mixer.forward(x.float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item()), (got - want).abs().max()
    # the same tokens in two steps, cut inside a page: the second step reads the pages of the first
    step = _step_for(runner, "b", 23)
    first = block.mixer.forward(x[:23].float().cuda(), step, runner.slots[0]).double().cpu()
    runner.cache.commit("b", 23)
    step = _step_for(runner, "b", n - 23, start=23)
    second = block.mixer.forward(x[23:].float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(torch.cat([first, second]), want, atol=2e-5 * want.abs().max().item())


def test_one_key_just_inside_and_just_outside_a_window(tmp_path):
    """Window 8, two kept tokens.  The value of token 5 is made huge: a query sees it while the
    token is within the window (queries 5 .. 12) and never after; token 1 is seen by everyone."""
    m = du.attention(2, 1, 16, 16, 8, base=50.0, scale=0.25, mask=(8, 2))
    runner, block, t = _one_layer(tmp_path, du.layer(m))
    torch.manual_seed(7)
    n = 30
    x = torch.randn(n, 56, dtype=F64)
    x[5] *= 50.0
    want = plain.attention_mixer(x, t, "l0.mix.", m, 1e-4)
    step = _step_for(runner, "a", n)
    got = block.mixer.forward(x.float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    inside, outside = want[12].abs().max().item(), want[13].abs().max().item()
    assert inside > 3 * outside        # the plain model itself sees the edge between queries 12 and 13


@pytest.mark.parametrize("e, top, groups, keep", [(8, 3, 4, 2), (6, 2, 3, 2), (1, 1, 1, 1), (9, 2, 3, 1), (64, 6, 8, 3),
                                                  (160, 8, 1, 1), (5, 5, 5, 5), (12, 3, 12, 4)])
def test_router(e, top, groups, keep):
    from qwen25vl_lite_amd.ops.moe import route
    torch.manual_seed(e)
    z = (2.0 * torch.randn(37, e)).float()
    ids, w = route(z.cuda(), top, groups, keep, scale=1.7)
    want_ids, want_w = plain.route(z.double(), top, groups, keep, 1.7)
    order = ids.cpu().long().sort(dim=1)
    assert torch.equal(order.values, want_ids.sort(dim=1).values)
    got_w = w.cpu().double().gather(1, order.indices)
    assert torch.allclose(got_w, want_w.gather(1, want_ids.sort(dim=1).indices), atol=1e-6)


@pytest.mark.parametrize("dtype, width, ff", [(torch.float32, 56, 24), (torch.bfloat16, 64, 40), (torch.bfloat16, 56, 24),
                                              (torch.bfloat16, 50, 11), (torch.float32, 50, 11), (torch.bfloat16, 128, 96),
                                              (torch.bfloat16, 96, 160)])
@pytest.mark.parametrize("rows", [3, 150, 700])
def test_routed_experts_alone(dtype, width, ff, rows, tmp_path):
    """Few rows (a tile of 16 pairs an expert) and many (one and several tiles of 128), widths on and off the matrix
    cores' steps and the steps of 32 that the kernel with fetches straight into LDS takes (a few and many of
    them), in float32 and bfloat16, with a shared expert and clamps that bite."""
    mlp = du.moe(6, 3, ff, 0.8, groups=(3, 2), scale=1.3, shared=(ff + 8, 0.5))
    lay = du.layer(du.attention(1, 1, 16, 16, 16, scale=0.25), mlp)
    runner, block, t = _one_layer(tmp_path, lay, dtype=dtype, width=width)
    torch.manual_seed(rows)
    x = torch.randn(rows, width).to(dtype)
    want = plain.moe(x.double(), t, "l0.mlp.", mlp)
    step = _step_for(runner, "a", min(rows, 256))
    got = block.ffn.forward(x.cuda(), step).double().cpu()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(got, want, atol=tol * want.abs().max().item()), (got - want).abs().max()
    ids, w = block.ffn.route(x.cuda())
    want_ids, _ = plain.route(x.double() @ t["l0.mlp.router"].T, 3, 3, 2, 1.3)
    assert torch.equal(ids.cpu().long().sort(1).values, want_ids.sort(1).values)


@pytest.mark.parametrize("width", [5, 72, 1000, 4100])
@pytest.mark.parametrize("ydtype", [torch.float32, torch.bfloat16])
def test_sum_and_norm_in_one_kernel(width, ydtype):
    from qwen25vl_lite_amd.ops.gated import sandwich_norm
    torch.manual_seed(width)
    n = 6
    h = torch.randn(n, width)
    y = (3 * torch.randn(n, width)).to(ydtype)
    gain, vec, w = torch.rand(width) + 0.5, torch.randn(width), torch.rand(width) + 0.5
    rows = torch.tensor([4, 1], dtype=torch.int32)
    added = h.double() + 0.3 * plain.rms_norm(y.double(), gain.double(), 1e-3) + vec.double()
    want = plain.rms_norm(added, w.double(), 1e-5)
    for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        hd = h.clone().cuda()
        picked = sandwich_norm(hd, y.cuda(), gain.cuda(), 1e-3, 0.3, vec.cuda(), w.cuda(), 1e-5, out_dtype, rows=rows.cuda())
        assert torch.equal(hd.cpu(), h)                                    # rows asked for: the sum is not written
        assert torch.allclose(picked.double().cpu(), want[rows.long()], atol=tol * 4, rtol=tol)
        out = sandwich_norm(hd, y.cuda(), gain.cuda(), 1e-3, 0.3, vec.cuda(), w.cuda(), 1e-5, out_dtype)
        assert torch.allclose(hd.double().cpu(), added, atol=1e-5)
        assert torch.allclose(out.double().cpu(), want, atol=tol * 4, rtol=tol)
    if ydtype == torch.float32:
        slabs = torch.randn(3, n, width)
        hd = h.clone().cuda()
        sandwich_norm(hd, slabs.cuda(), None, 0.0, 1.0, None, None, 0.0, torch.float32)      # a plain sum of slabs
        assert torch.allclose(hd.double().cpu(), h.double() + slabs.double().sum(0), atol=1e-5)


# ---------------------------------------------------------------------------------------------
# whole models, every schedule
# ---------------------------------------------------------------------------------------------
LENGTHS = {"a": 77, "b": 1, "c": 34, "d": 2, "e": 120, "f": 19}


def _requests(vocab, seed=0):
    return {rid: random_tokens(n, vocab, seed + i) for i, (rid, n) in enumerate(LENGTHS.items())}


@pytest.mark.parametrize("name", ["mixed", "ones", "odd"])
def test_float32_every_schedule_against_the_plain_model(name, folders):
    """Whole prompts, decoded tails, portions down to two tokens, mixed batches with more requests
    than slots: all the same logits, and the plain model's."""
    folder = folders[name]
    cfg, _ = plain.dazapel_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=20)
    want = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    mixed, peak = mixed_trace(reqs, seed=4, max_live=4)
    holders = {}
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 50), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "float32", size), steps, holders if steps is mixed else None)
        for rid, toks in reqs.items():
            assert _rel(_rows(got, rid, len(toks)), want[rid]) < 2e-5, (name, rid)
    assert any(len(who) > 1 for who in holders.values()), "no page was used by two requests"


@pytest.mark.parametrize("name", ["mixed", "ones", "odd"])
def test_bfloat16_within_rounding_of_the_plain_model(name, folders):
    """bfloat16 kernels: no further from exact arithmetic than rounding the stored activations to
    bfloat16 takes the plain model, whatever the schedule."""
    folder = folders[name]
    cfg, _ = plain.dazapel_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=30)
    exact = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    rounding = torch.cat([_rel_rows(_oracle(folder, toks, plain.to_bfloat16_and_back), exact[rid])
                          for rid, toks in reqs.items()])
    mixed, peak = mixed_trace(reqs, seed=5, max_live=4)
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 50), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "bfloat16", size), steps)
        errors = torch.cat([_rel_rows(_rows(got, rid, len(toks)), exact[rid]) for rid, toks in reqs.items()])
        assert _like_rounding(errors, rounding), (name, errors.median(), rounding.median(), errors.quantile(0.9),
                                                  rounding.quantile(0.9))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_peaked_attention_at_window_edges_kept_tokens_and_far_keys(dtype, folders):
    """Score scales so large that the softmax picks single keys: in the layer that sees everything,
    hundreds of tokens back and across page borders; in the windowed ones, right at the window's edge and
    among the kept first tokens.  The last 70 tokens are decoded, so every window (9, 21, 37) passes
    over decoded tokens; then the same in portions."""
    folder = folders["sharp"]
    toks = random_tokens(330, du.SHARP["vocab"], 40)
    want = _oracle(folder, toks)
    rounding = _rel_rows(_oracle(folder, toks, plain.to_bfloat16_and_back), want)
    for steps in (tail_trace({"s": toks}, 70), portion_trace({"s": toks}, (64, 3, 41, 2, 17, 90))):
        got = _rows(run_steps(_replayer(folder, dtype, round64(len(toks))), steps), "s", len(toks))
        if dtype == "float32":
            assert _rel(got, want) < 2e-5
        else:
            errors = _rel_rows(got, want)
            assert _like_rounding(errors, rounding), (errors.median(), rounding.median(), errors.quantile(0.9),
                                                      rounding.quantile(0.9))


def test_sharpening_matters(folders):
    """The test above would see a window that is one token off, a lost kept token, or a lost far key:
    each changes the plain model's last logits."""
    toks = random_tokens(330, du.SHARP["vocab"], 40)
    whole = _oracle(folders["sharp"], toks)[-30:]

    def one_off(cfg):
        for lay in cfg["layers"]:
            if lay["mixer"].get("mask"):
                lay["mixer"]["mask"]["size"] -= 1

    def fewer_kept(cfg):
        for lay in cfg["layers"]:
            if lay["mixer"].get("mask") and lay["mixer"]["mask"]["keep_first"]:
                lay["mixer"]["mask"]["keep_first"] -= 1

    def nothing_far(cfg):
        cfg["layers"][2]["mixer"]["mask"] = {"size": 200, "keep_first": 0}

    for edit in (one_off, fewer_kept, nothing_far):
        assert _rel(_oracle(folders["sharp"], toks, cfg_edit=edit)[-30:], whole) > 0.02, edit.__name__


def test_long_decoding(folders):
    """A short prompt and 200 tokens decoded one by one, through several pages, windows moving on."""
    folder = folders["mixed"]
    toks = random_tokens(205, du.MIXED["vocab"], 50)
    want = _oracle(folder, toks)
    got = _rows(run_steps(_replayer(folder, "float32", 256), tail_trace({"l": toks}, 200)), "l", len(toks))
    assert _rel(got, want) < 2e-5


def test_windowed_groups_give_pages_back_while_decoding(folders):
    from qwen25vl_lite_amd.engine.replay import Replayer
    rp = Replayer(folders["mixed"], "float32", 256, 16, 2)
    toks = random_tokens(200, du.MIXED["vocab"], 51)
    run_steps(rp, [{"step": 0, "entries": [{"id": "x", "tokens": toks, "want": []}], "end": []}])
    cache = rp.runner.cache
    held = {(g.need.window, g.need.keep_first): sum(p >= 0 for p in cache.table("x", i)) for i, g in enumerate(cache.groups)}
    assert held[(None, 0)] == 13 and held[(9, 3)] == 1 + 1 and held[(21, 0)] == 2 and held[(37, 18)] == 2 + 3
    rp.step({"entries": [], "end": ["x"]})
    cache.check()


@pytest.mark.parametrize("graph", [False, True])
def test_greedy_generation_through_the_entry_point(graph, folders):
    """``LLM.generate`` with the scheduler (three prompts, two slots, portions of 16 tokens, decode
    steps from HIP graphs or not) picks the plain model's tokens."""
    from qwen25vl_lite_amd import LLM, SamplingParams
    folder = folders["mixed"]
    prompts = [random_tokens(n, du.MIXED["vocab"], 70 + n) for n in (37, 5, 21)]
    steps = 12
    want = []
    for p in prompts:
        ids = list(p)
        for _ in range(steps):
            ids.append(int(torch.argmax(_oracle(folder, ids)[-1])))
        want.append(ids[len(p):])
    with LLM(folder, dtype="float32", num_blocks=32, block_size=16, max_num_seqs=2, max_num_batched_tokens=16,
             hip_graph=graph) as llm:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))
    assert [o.output_token_ids for o in outs] == want


def test_bfloat16_generation_from_graphs_matches_eager_steps(folders):
    from qwen25vl_lite_amd import LLM, SamplingParams
    prompts = [random_tokens(n, du.MIXED["vocab"], 90 + n) for n in (18, 3, 40, 9)]
    outs = []
    for graph in (False, True):
        with LLM(folders["mixed"], dtype="bfloat16", num_blocks=48, block_size=16, max_num_seqs=4,
                 max_num_batched_tokens=64, hip_graph=graph) as llm:
            outs.append([o.output_token_ids for o in
                         llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))])
    assert outs[0] == outs[1]


# ---------------------------------------------------------------------------------------------
# the matrix-core attention for windows that keep the first keys
# ---------------------------------------------------------------------------------------------
def _paged_case(runs, hd, vd, nkv, ps, seed):
    """Requests of (tokens already cached, tokens in this step): keys and values in shuffled pages."""
    import types
    g = torch.Generator().manual_seed(seed)
    ctx = [a + b for a, b in runs]
    need = [(c + ps - 1) // ps for c in ctx]
    perm = torch.randperm(sum(need) + 3, generator=g).tolist()
    width = max(need)
    table = torch.full((len(runs), width), -1, dtype=torch.int32)
    k_cache = torch.zeros(sum(need) + 3, nkv, ps, hd)
    v_cache = torch.zeros(sum(need) + 3, nkv, vd, ps)
    keys, values = [], []
    for r, c in enumerate(ctx):
        k, v = torch.randn(c, nkv, hd, generator=g), torch.randn(c, nkv, vd, generator=g)
        keys.append(k.to(torch.bfloat16).float())
        values.append(v.to(torch.bfloat16).float())
        for i in range(need[r]):
            page = perm.pop()
            table[r, i] = page
            n = min(ps, c - i * ps)
            k_cache[page, :, :n] = keys[r][i * ps:i * ps + n].transpose(0, 1)
            v_cache[page, :, :, :n] = values[r][i * ps:i * ps + n].permute(1, 2, 0)
    cu = [0]
    for _, b in runs:
        cu.append(cu[-1] + b)
    step = types.SimpleNamespace(
        num_reqs=len(runs), cu_q=torch.tensor(cu, dtype=torch.int32).cuda(), ctx_len=torch.tensor(ctx, dtype=torch.int32).cuda(),
        cu_q_host=cu, ctx_len_host=ctx, max_q_len=max(b for _, b in runs), max_ctx_len=max(ctx), derived={})
    return step, table.cuda(), k_cache.to(torch.bfloat16).cuda(), v_cache.to(torch.bfloat16).cuda(), keys, values


@pytest.mark.parametrize("hd, vd, nq, nkv, ps", [(16, 24, 4, 2, 16), (48, 16, 3, 1, 16), (128, 128, 8, 2, 16), (64, 32, 20, 1, 8),
                                                 (16, 16, 2, 2, 48)])
@pytest.mark.parametrize("window, keep", [(9, 3), (37, 18), (70, 0), (33, 100), (None, 0)])
def test_window_attention_on_the_matrix_cores(hd, vd, nq, nkv, ps, window, keep):
    """Prompt portions that start anywhere and decoded tokens, a wave per tile and four waves sharing a tile,
    against dense masked attention: windows that end inside a block of keys, kept keys that reach into
    the window, pages in shuffled order."""
    from qwen25vl_lite_amd.ops.attention_window import try_attention
    for runs in ([(0, 75), (130, 1), (37, 2), (95, 41), (0, 1)], [(199, 1), (64, 1), (3, 1)]):
        step, table, kc, vc, keys, values = _paged_case(runs, hd, vd, nkv, ps, seed=hd + (window or 0))
        n = step.cu_q_host[-1]
        q = torch.randn(n, nq, hd, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
        scale = 2.0 * hd ** -0.5
        want = torch.empty(n, nq, vd)
        for r, (before, now) in enumerate(runs):
            see = plain.visible(before + now, window, keep)[before:]
            for h in range(nq):
                s = (q[step.cu_q_host[r]:step.cu_q_host[r + 1], h].float() @ keys[r][:, h // (nq // nkv)].T) * scale
                want[step.cu_q_host[r]:step.cu_q_host[r + 1], h] = torch.softmax(s.masked_fill(~see, float("-inf")), -1) @ values[r][:, h // (nq // nkv)]
        for share in (False, True):
            got = try_attention(q.reshape(n, nq * hd).cuda(), kc, vc, table, step, nq, window, keep, scale, share=share)
            assert got is not None
            assert torch.allclose(got.float().cpu().view(n, nq, vd), want, atol=2e-2, rtol=2e-2), (runs, share)
