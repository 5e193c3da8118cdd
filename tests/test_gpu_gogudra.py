"""The Gogudra decoder on the GPU against the plain implementation in ``plain_gogudra.py``: each
mechanism alone, whole prompts, decoding, portions, mixed batches, pages and slots used again,
peaked attention over far keys, sizes that are 1 or equal, and greedy generation through ``LLM``."""

import copy

import pytest
import torch

import gogudra_util as gu
import plain_gogudra as plain
from replay_util import mixed_trace, portion_trace, random_tokens, round64, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu

F64 = torch.float64


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg, seed, rank, sharp in (("mixed", gu.MIXED, 11, 6, 1.0), ("sharp", gu.MIXED, 12, 6, 6.0),
                                         ("ones", gu.ONES, 13, 3, 2.0), ("no_pages", gu.NO_PAGES, 14, 10, 1.0),
                                         ("odd", gu.ODD, 15, 5, 1.0)):
        out[name] = gu.write_model(str(tmp_path_factory.mktemp(name)), cfg, seed, rank, sharp)
    return out


def _oracle(folder, tokens, store=None):
    cfg, tensors = plain.gogudra_read(folder, F64)
    return plain.gogudra_logits(cfg, tensors, tokens, store or plain._keep).to(torch.float32)


def _rel(got, want):
    """Per row: RMS of the difference (mean taken off) over the RMS of the wanted row."""
    d = (got - want).double()
    d = d - d.mean(dim=1, keepdim=True)
    return (d.pow(2).mean(dim=1).sqrt() / want.double().pow(2).mean(dim=1).sqrt()).max().item()


def _replayer(folder, dtype, max_tokens, max_live=4):
    from qwen25vl_lite_amd.engine.replay import Replayer
    return Replayer(folder, dtype, max_tokens, 16, max_live)


def _rows(got, rid, n):
    return torch.stack([got[(rid, p)] for p in range(n)])


# ---------------------------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------------------------
def _one_layer(tmp_path, layer, rank=4, seed=0, width=56):
    """A one-layer model around the mixer under test; returns (runner, mixer, its tensors in float64)."""
    from qwen25vl_lite_amd.config import EngineConfig, load_config
    from qwen25vl_lite_amd.engine import ModelRunner
    from qwen25vl_lite_amd.models import build_model
    from qwen25vl_lite_amd.weights import load_weights
    cfg = gu.config(width, 50, [layer], eps=1e-4)
    d = gu.write_model(str(tmp_path / "one"), cfg, seed, rank)
    model = build_model(load_config(d), torch.float32, "cuda:0")
    load_weights(d, model)
    ecfg = EngineConfig(num_blocks=16, block_size=16, max_num_seqs=3, max_num_batched_tokens=256, max_model_len=256,
                        enable_prefix_cache=False, dtype=torch.float32)
    _, tensors = plain.gogudra_read(d, F64)
    return ModelRunner(model, ecfg), model.blocks[0], plain._sub(tensors, "l0.mix."), plain._sub(tensors, "l0.mlp.")


def _step_for(runner, rid, n, start=0):
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.engine.batch import build_step
    if start == 0:
        runner.admit(rid)
    e = StepEntry(rid, [0] * n, start)
    runner.cache.reserve(rid, start + n)
    runner._clear_state([e])
    step = build_step([e], runner.cache, 1, torch.float32, runner.device)
    return step


@pytest.mark.parametrize("kind", ["lightning", "gla", "attention"])
def test_a_mixer_alone_whole_and_in_two_steps(kind, tmp_path):
    layer = {"lightning": gu.lightning_layer(3, 20, 24, [0.3, 0.9, 1.0]),
             "gla": gu.gla_layer(2, 12, 40, 2.5),
             "attention": gu.attention_layer(4, 2, 20, 12, base=300.0, scale=0.45,
                                             scaling={"factor": 4.0, "low": 1.0, "high": 3.0, "original": 24})}[kind]
    runner, block, w, _ = _one_layer(tmp_path, layer)
    torch.manual_seed(5)
    t = 41
    x = torch.randn(t, 56, dtype=F64)
    want = plain.MIXERS[kind](x, w, layer["mixer"], 1e-4)
    step = _step_for(runner, "a", t)
    got = block.mixer.forward(x.float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item()), (got - want).abs().max()
    # the same tokens in two steps, cut inside a page: the second step starts from the pages or state of the first
    step = _step_for(runner, "b", 23)
    first = block.mixer.forward(x[:23].float().cuda(), step, runner.slots[0]).double().cpu()
    runner.cache.commit("b", 23)
    step = _step_for(runner, "b", t - 23, start=23)
    second = block.mixer.forward(x[23:].float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(torch.cat([first, second]), want, atol=2e-5 * want.abs().max().item())


def test_decay_of_one_channel_reaches_far_back(tmp_path):
    """One key channel of a gated-linear head is made to remember (its decay's bias is large) and to
    carry a large key at token 3 only; the value written then must still be read 150 tokens later."""
    layer = gu.gla_layer(1, 8, 8, 1.0)
    runner, block, w, _ = _one_layer(tmp_path, layer, rank=2)
    mixer = block.mixer
    t, hidden = 160, 56
    torch.manual_seed(6)
    x = 0.05 * torch.randn(t, hidden, dtype=F64)
    x[3] += 2.0 * w["k"][0] / w["k"][0].norm()          # token 3 has a large key in channel 0
    x[155] += 2.0 * w["q"][0] / w["q"][0].norm()        # token 155 asks for channel 0
    w = dict(w)
    w["a2.b"] = w["a2.b"].clone()
    w["a2.b"][0] = 12.0                                  # channel 0 forgets almost nothing
    mixer.b_a2.copy_(w["a2.b"].float())
    want = plain.gla_mixer(x, w, layer["mixer"], 1e-4)
    forgetful = dict(w, **{"a2.b": w["a2.b"].clone()})
    forgetful["a2.b"][0] = -3.0
    assert (plain.gla_mixer(x, forgetful, layer["mixer"], 1e-4)[155] - want[155]).abs().max() > 0.05 * want[155].abs().max()
    step = _step_for(runner, "a", t)
    got = mixer.forward(x.float().cuda(), step, runner.slots[0]).double().cpu()
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())


def test_feed_forward_clamps(tmp_path):
    """Inputs large enough that both clamps act, on both sides of the linear branch."""
    layer = gu.lightning_layer(1, 8, 8, [0.5], gu.dense(72, 0.6))
    runner, block, _, w = _one_layer(tmp_path, layer)
    torch.manual_seed(7)
    x = 3.0 * torch.randn(9, 56, dtype=F64)
    g, u = x @ w["gate"].T, x @ w["up"].T
    assert (g > 0.6).any() and (u > 0.6).any() and (u < -0.6).any() and (g < -0.6).any()
    want = plain.clamped_gated_ff(x, w, layer["mlp"])
    got = block.ffn.forward(x.float().cuda(), None).double().cpu()
    assert torch.allclose(got, want, atol=1e-5 * want.abs().max().item())


def test_norm_with_weight_around_zero_and_capped_head():
    from qwen25vl_lite_amd.parts import PartSpec, ResidualStream, build_part
    dev = torch.device("cuda:0")
    torch.manual_seed(8)
    norm = build_part("norm", PartSpec("rms_norm", {"size": 52, "eps": 1e-2, "offset": 1.0}), torch.float32, dev)
    w = 0.2 * torch.randn(52)
    norm.load({"weight": w.cuda()})
    h, d = torch.randn(5, 52), 0.01 * torch.randn(5, 52)
    out = norm.forward(ResidualStream(h.cuda(), d.cuda())).cpu()
    assert torch.allclose(out, plain.layer_norm_one_plus((h + d).double(), w.double(), 1e-2).float(), atol=1e-5)
    head = build_part("head", PartSpec("linear", {"vocab_size": 33, "hidden_size": 52, "softcap": 2.5}), torch.float32, dev)
    table = torch.randn(33, 52)
    head.load({"weight": table.cuda()})
    x = torch.randn(4, 52)
    want = 2.5 * torch.tanh((x.double() @ table.double().T) / 2.5)
    assert (x @ table.T).abs().max() > 5 and torch.allclose(head.forward(x.cuda(), None).cpu().double(), want, atol=1e-5)


def test_rotation_pairs_neighbouring_channels():
    """The kernel that norms, rotates and writes: interleaved pairs on the first channels only, the
    value written is the key before norm and rotation."""
    from qwen25vl_lite_amd.ops import gated, kernels
    torch.manual_seed(9)
    n, nq, nkv, hd, rot, ps = 19, 3, 1, 12, 8, 16
    x = torch.randn(n, (nq + nkv) * hd + 5)
    qw, kw = 1 + 0.2 * torch.randn(hd), 1 + 0.2 * torch.randn(hd)
    freqs = [0.9, 0.31, 0.07, 0.011]
    pos = torch.arange(100, 100 + n, dtype=torch.int32)
    cs = kernels.rope_table(pos[None].cuda(), torch.tensor(freqs).cuda(), torch.zeros(4, dtype=torch.int32).cuda(), n)
    kc = torch.zeros(3, nkv, ps, hd).cuda()
    vc = torch.zeros(3, nkv, hd, ps).cuda()
    slots = (torch.arange(n, dtype=torch.int32) + 20).cuda()      # pages 1 and 2
    q = gated.qk_norm_rope_write(x.cuda(), qw.cuda(), kw.cuda(), 1e-3, cs, slots, kc, vc, nq, nkv, hd, ps, torch.float32,
                                 interleaved=True, values_are_keys=True).cpu()
    xq = x[:, :nq * hd].view(n, nq, hd).double()
    xk = x[:, nq * hd:(nq + nkv) * hd].view(n, nkv, hd).double()
    want_q = plain.rotate_interleaved(plain.unit_rms(xq, 1e-3) * qw.double(), pos, freqs)
    want_k = plain.rotate_interleaved(plain.unit_rms(xk, 1e-3) * kw.double(), pos, freqs)
    assert torch.allclose(q.view(n, nq, hd).double(), want_q, atol=1e-5)
    assert torch.equal(want_q[..., rot:], plain.unit_rms(xq, 1e-3)[..., rot:] * qw.double()[rot:])
    flat_k = kc.cpu().permute(0, 2, 1, 3).reshape(3 * ps, nkv, hd)[20:20 + n]
    flat_v = vc.cpu().permute(0, 3, 1, 2).reshape(3 * ps, nkv, hd)[20:20 + n]
    assert torch.allclose(flat_k.double(), want_k, atol=1e-5) and torch.equal(flat_v.double(), xk)


# ---------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------
LENGTHS = {"a": 70, "b": 33, "c": 1, "d": 2, "e": 49, "f": 18}


def _requests(vocab, seed=0):
    return {rid: random_tokens(n, vocab, seed + i) for i, (rid, n) in enumerate(LENGTHS.items())}


@pytest.mark.parametrize("name", ["mixed", "ones", "no_pages"])
def test_float32_every_schedule_against_the_plain_model(name, folders):
    """Whole prompts, decoded tails, portions down to two tokens, mixed batches with more requests
    than slots: all the same logits, and the plain model's."""
    folder = folders[name]
    cfg, _ = plain.gogudra_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=20)
    want = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    mixed, peak = mixed_trace(reqs, seed=4, max_live=4)
    holders = {}
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 20), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "float32", size), steps, holders if steps is mixed else None)
        for rid, toks in reqs.items():
            rows = _rows(got, rid, len(toks))
            assert _rel(rows, want[rid]) < 2e-5, (name, rid)
    if cfg and any(l["type"] == "attention" for l in cfg["layers"]):
        assert any(len(who) > 1 for who in holders.values()), "no page was used by two requests"


@pytest.mark.parametrize("name", ["mixed", "ones"])
def test_bfloat16_within_rounding_of_the_plain_model(name, folders):
    """bfloat16 kernels: no further from exact arithmetic than three times what rounding the
    stored activations to bfloat16 costs the plain model, whatever the schedule."""
    folder = folders[name]
    cfg, _ = plain.gogudra_read(folder, F64)
    reqs = _requests(cfg["vocab"], seed=30)
    exact = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    rounded = max(_rel(_oracle(folder, toks, plain.to_bfloat16_and_back), exact[rid]) for rid, toks in reqs.items())
    mixed, peak = mixed_trace(reqs, seed=5, max_live=4)
    for steps, size in ((whole_trace(reqs), 128), (tail_trace(reqs, 20), 128), (portion_trace(reqs), 128), (mixed, peak)):
        got = run_steps(_replayer(folder, "bfloat16", size), steps)
        for rid, toks in reqs.items():
            assert _rel(_rows(got, rid, len(toks)), exact[rid]) < 3 * rounded, (name, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_peaked_attention_over_far_keys_and_page_borders(dtype, folders):
    """Query norm weights scaled up: the softmax picks single keys, near and hundreds of tokens
    back, so one wrong key, page or position moves the logits.  The last 40 tokens are decoded."""
    folder = folders["sharp"]
    toks = random_tokens(330, gu.MIXED["vocab"], 40)
    want = _oracle(folder, toks)
    rp = _replayer(folder, dtype, round64(len(toks)))
    got = _rows(run_steps(rp, tail_trace({"s": toks}, 40)), "s", len(toks))
    bound = 2e-5 if dtype == "float32" else 3 * _rel(_oracle(folder, toks, plain.to_bfloat16_and_back), want)
    assert _rel(got, want) < bound


def test_sharpening_matters(folders):
    """The test above would see a lost key: dropping the first 200 tokens changes the last logits."""
    toks = random_tokens(330, gu.MIXED["vocab"], 40)
    whole = _oracle(folders["sharp"], toks)[-1:]
    cut = _oracle(folders["sharp"], toks[200:])[-1:]
    assert _rel(cut, whole) > 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_odd_sizes_and_a_long_prompt(dtype, folders):
    """Sizes that no vector width divides, in a prompt long enough for the chunked recurrence, whole and in portions."""
    folder = folders["odd"]
    reqs = {"o": random_tokens(150, gu.ODD["vocab"], 80), "p": random_tokens(3, gu.ODD["vocab"], 81)}
    want = {rid: _oracle(folder, toks) for rid, toks in reqs.items()}
    bound = 2e-5 if dtype == "float32" else 3 * max(
        _rel(_oracle(folder, toks, plain.to_bfloat16_and_back), want[rid]) for rid, toks in reqs.items())
    for steps in (whole_trace(reqs), portion_trace(reqs, (130, 2, 5, 13))):
        got = run_steps(_replayer(folder, dtype, 256), steps)
        for rid, toks in reqs.items():
            assert _rel(_rows(got, rid, len(toks)), want[rid]) < bound, (dtype, rid)


def test_long_decoding(folders):
    """A short prompt and 200 tokens decoded one by one, through several pages."""
    folder = folders["mixed"]
    toks = random_tokens(205, gu.MIXED["vocab"], 50)
    want = _oracle(folder, toks)
    got = _rows(run_steps(_replayer(folder, "float32", 256), tail_trace({"l": toks}, 200)), "l", len(toks))
    assert _rel(got, want) < 2e-5


def test_a_slot_used_again_starts_from_zero(folders):
    """One state slot: the second request must not see what the first left in it."""
    folder = folders["no_pages"]
    a, b = random_tokens(30, 64, 60), random_tokens(12, 64, 61)
    rp = _replayer(folder, "float32", 64, max_live=1)
    got = run_steps(rp, whole_trace({"a": a, "b": b}))
    assert _rel(_rows(got, "b", len(b)), _oracle(folder, b)) < 2e-5


@pytest.mark.parametrize("graph", [False, True])
def test_greedy_generation_through_the_entry_point(graph, folders):
    """``LLM.generate`` with the scheduler (three prompts, two slots, portions of 16 tokens, decode
    steps from HIP graphs or not) picks the plain model's tokens."""
    from qwen25vl_lite_amd import LLM, SamplingParams
    folder = folders["mixed"]
    prompts = [random_tokens(n, gu.MIXED["vocab"], 70 + n) for n in (37, 5, 21)]
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


def test_scan_cut_into_groups_of_key_channels():
    """Long runs are spread over more blocks by cutting the key channels into groups whose partial
    outputs are added afterwards: the same outputs and the same final state."""
    from qwen25vl_lite_amd.ops.linear_attention import decayed_scan, scan_groups
    assert scan_groups(1, 512, 4, 64, 64, "cuda:0") > 1 and scan_groups(8, 1, 4, 64, 64, "cuda:0") == 1
    torch.manual_seed(10)
    n, h, d, v = 150, 2, 32, 72
    proj = torch.randn(n, 2 * h * d + h * v + 3).cuda()
    z = (2 + torch.randn(n, h * d)).cuda()
    cu = torch.tensor([0, 90, 150], dtype=torch.int32).cuda()
    slots = torch.tensor([2, 0], dtype=torch.int32).cuda()
    outs, states = [], []
    for groups in (1, 2, 8):
        state = torch.zeros(3, h, d, v).cuda()
        o = decayed_scan(proj, 0, h * d, 2 * h * d, h, d, v, state, cu, slots, z=z, tau=3.0, q_scale=0.5, groups=groups)
        assert o.shape == (groups, n, h * v)
        outs.append(o.sum(0).cpu())
        states.append(state.cpu())
    q, k, vv = proj[:, :h * d].cpu().double(), proj[:, h * d:2 * h * d].cpu().double(), proj[:, 2 * h * d:2 * h * d + h * v].cpu().double()
    decay = torch.exp(torch.nn.functional.logsigmoid(z.cpu().double()) / 3.0)
    for head in range(h):
        sl, sv = slice(head * d, (head + 1) * d), slice(head * v, (head + 1) * v)
        want, s_end = plain.decayed_outer_product_scan(0.5 * q[:90, sl], k[:90, sl], vv[:90, sv], decay[:90, sl])
        for o, st in zip(outs, states):
            assert torch.allclose(o[:90, sv].double(), want, atol=1e-4 * want.abs().max().item())
            assert torch.allclose(st[2, head].double(), s_end, atol=1e-4 * s_end.abs().max().item())
            assert st[1].abs().max() == 0


def test_a_large_key_size():
    """Keys of 320 channels: fewer tokens are staged at a time and the decays' prefix is not cut."""
    from qwen25vl_lite_amd.ops.linear_attention import chunked_scan, decayed_scan, plan_chunks
    torch.manual_seed(12)
    n, h, d, v = 130, 1, 320, 24
    proj = (0.2 * torch.randn(n, 2 * h * d + h * v)).cuda()
    z = (3 + torch.randn(n, h * d)).cuda()
    cu = torch.tensor([0, n], dtype=torch.int32).cuda()
    slots = torch.tensor([0], dtype=torch.int32).cuda()
    s1 = torch.zeros(1, h, d, v).cuda()
    got = decayed_scan(proj, 0, h * d, 2 * h * d, h, d, v, s1, cu, slots, z=z, tau=1.5).sum(0).cpu().double()
    p = proj.cpu().double()
    decay = torch.exp(torch.nn.functional.logsigmoid(z.cpu().double()) / 1.5)
    want, s_end = plain.decayed_outer_product_scan(p[:, :d], p[:, d:2 * d], p[:, 2 * d:], decay)
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item())
    assert torch.allclose(s1[0, 0].cpu().double(), s_end, atol=2e-5 * s_end.abs().max().item())
    s2 = torch.zeros(1, h, d, v).cuda()
    cut = chunked_scan(proj, 0, h * d, 2 * h * d, h, d, v, s2, plan_chunks([0, n], "cuda:0"), slots, z=z, tau=1.5)
    assert torch.allclose(cut.sum(0).cpu().double(), want, atol=2e-5 * want.abs().max().item())


@pytest.mark.parametrize("channel", [False, True])
def test_long_runs_scanned_in_chunks(channel):
    """Runs cut into chunks that are scanned side by side and stitched through the carried state: the
    same outputs and final states as one scan, for runs that end inside a chunk, a run of one token,
    and states that do not start at zero."""
    from qwen25vl_lite_amd.ops.linear_attention import chunked_scan, decayed_scan, plan_chunks
    torch.manual_seed(11)
    runs = [150, 1, 64, 70]
    n, h, d, v = sum(runs), 3, 16, 40
    proj = torch.randn(n, 2 * h * d + h * v).cuda()
    z = (1 + 2 * torch.randn(n, h * d)).cuda() if channel else None
    decay = None if channel else torch.tensor([0.5, 0.97, 1.0]).cuda()
    bounds = [0]
    for r in runs:
        bounds.append(bounds[-1] + r)
    cu = torch.tensor(bounds, dtype=torch.int32).cuda()
    slots = torch.tensor([3, 0, 1, 2], dtype=torch.int32).cuda()
    start = 0.3 * torch.randn(5, h, d, v).cuda()
    how = dict(head_decay=decay, z=z, tau=2.0, silu=not channel, q_scale=0.7)
    s1 = start.clone()
    want = decayed_scan(proj, 0, h * d, 2 * h * d, h, d, v, s1, cu, slots, **how).sum(0)
    s2 = start.clone()
    plan = plan_chunks(bounds, "cuda:0", 64)
    assert plan.chunks == 3 + 1 + 1 + 2 and plan.req_first.tolist() == [0, 3, 4, 5, 7]
    got = chunked_scan(proj, 0, h * d, 2 * h * d, h, d, v, s2, plan, slots, **how).sum(0)
    assert torch.allclose(got, want, atol=2e-5 * want.abs().max().item()), (got - want).abs().max()
    assert torch.allclose(s2, s1, atol=2e-5 * s1.abs().max().item()) and torch.equal(s2[4], start[4])


@pytest.mark.parametrize("span, groups", [(7, 3), (24, 5), (128, 2), (1024, 1), (1500, 2), (4100, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_group_norm_with_gate_at_any_width(span, groups, dtype):
    """Narrow groups (a wave each), wide ones (a block each), widths that are not a multiple of four,
    partial sums in slabs, a gate that is a view of a wider tensor."""
    from qwen25vl_lite_amd.ops.gated import group_norm_gate
    torch.manual_seed(span)
    n, c = 5, span * groups
    slabs = torch.randn(3, n, c)
    wide = torch.randn(n, c + 8).to(dtype)
    for weight in (torch.randn(span), torch.randn(c)):
        for act, fn in (("sigmoid", torch.sigmoid), ("silu", torch.nn.functional.silu)):
            x = slabs.sum(0).double().view(n, groups, span)
            want = (plain.unit_rms(x, 1e-3).view(n, c) * weight.double().repeat(c // weight.shape[0])
                    * fn(wide[:, 8:].double()))
            got = group_norm_gate(slabs.cuda(), weight.cuda(), span, 1e-3, dtype, gate=wide.cuda()[:, 8:], gate_act=act)
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            assert torch.allclose(got.double().cpu(), want, atol=tol * want.abs().max().item(), rtol=tol)


@pytest.mark.parametrize("inter", [5, 72, 1000])
def test_gated_activation_at_any_width(inter):
    from qwen25vl_lite_amd.ops.gated import gated_act
    torch.manual_seed(inter)
    x = 2 * torch.randn(7, 2 * inter)
    for dtype in (torch.float32, torch.bfloat16):
        xd = x.to(dtype)
        g, u = xd[:, :inter].double().clamp(max=0.9), xd[:, inter:].double().clamp(-0.9, 0.9)
        want = g * torch.sigmoid(1.3 * g) * (u + 0.5)
        got = gated_act(xd.cuda(), 1.3, 0.9, 0.5).double().cpu()
        assert torch.allclose(got, want, atol=1e-5 if dtype == torch.float32 else 2e-2)
        free = gated_act(xd.cuda()).double().cpu()
        assert torch.allclose(free, torch.nn.functional.silu(xd[:, :inter].double()) * xd[:, inter:].double(),
                              atol=1e-5 if dtype == torch.float32 else 1e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)
