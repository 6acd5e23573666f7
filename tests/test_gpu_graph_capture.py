"""The kernels under HIP graph capture: a captured micro-step is replayed on new inputs several times, with eager
work and synchronisations between the replays, and every replay must equal the eager result bit for bit (the same
kernels run in both).  Three graphs: log-prob kernel -> GRPO loss through the entry point that allocates nothing ->
gradient kernel; the single-pass GRPO kernel; the fused head forward (products kept) and backward, bf16 and fp16.  The library records no memset into a graph and keeps no host
state between launches, which is what these replays would show if it did."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
B, T, V = 6, 40, 4096


def _new_inputs(buf, seed):
    """Fills the static input buffers in place (eagerly) with the problem of this seed."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    buf["logits"].copy_((2.0 * torch.randn((B, T + 1, V), generator=g, device=DEV)).bfloat16())
    buf["ids"].copy_(torch.randint(0, V, (B, T), generator=g, device=DEV))
    lengths = torch.randint(0, T + 1, (B,), generator=g, device=DEV)
    buf["mask"].copy_((torch.arange(T, device=DEV)[None] < lengths[:, None]).float())
    buf["adv"].copy_(torch.randn((B,), generator=g, device=DEV))
    buf["old_noise"].copy_(0.05 * torch.randn((B, T), generator=g, device=DEV))
    buf["n_items"].copy_(buf["mask"].sum().clamp(min=1.0).reshape(1))


def _buffers():
    return dict(
        logits=torch.zeros((B, T + 1, V), dtype=torch.bfloat16, device=DEV), ids=torch.zeros((B, T), dtype=torch.int64, device=DEV),
        mask=torch.zeros((B, T), device=DEV), adv=torch.zeros((B,), device=DEV), old_noise=torch.zeros((B, T), device=DEV),
        n_items=torch.ones((1,), device=DEV), loss=torch.zeros((), device=DEV), metrics=torch.zeros((16,), device=DEV),
        dlogp=torch.zeros((B, T), device=DEV), row_scale=torch.zeros((B,), device=DEV))


def _two_pass_step(buf):
    from trl_amd import _lib, ops

    idx = buf["ids"].reshape(B * T, 1)
    lp, ent, lse = ops.logp_entropy_fwd(buf["logits"], idx, 0.9, 0, T, None)
    lp2 = lp.view(B, T)
    old = lp2 + buf["old_noise"]
    ops.grpo_loss_static_(buf["loss"], buf["metrics"], buf["dlogp"], None, lp2, old, None, ent.view(B, T), buf["adv"], buf["mask"],
                          None, None, buf["n_items"], _lib.DAPO, 0.2, 0.28, math.nan, 0.0, False, 1.0, float(B * T), 1.0, 0.0)
    dlogits = ops.logp_entropy_bwd(buf["logits"], idx, 0.9, 0, T, lse, None, buf["dlogp"].view(B * T, 1), None)
    return lp, ent, buf["loss"], buf["metrics"], dlogits


def _single_pass_step(buf):
    from trl_amd import _lib, ops

    buf["row_scale"].copy_((1.0 / buf["n_items"]).expand(B))  # dapo: 1 / num_items for every sequence
    return ops.grpo_fused_fwd_bwd(buf["logits"], buf["ids"], 0.9, 0, T, buf["mask"], buf["adv"], buf["row_scale"], None, None,
                                  None, None, _lib.TERM_CLIP, 0.2, 0.28, math.nan, 0.0, False, 1.0, 1.05)


@pytest.mark.parametrize("step", [_two_pass_step, _single_pass_step], ids=["two_pass", "single_pass"])
def test_graph_replays_equal_eager(step):
    from trl_amd import _lib

    assert _lib.lib.trlk_init() == 0
    buf = _buffers()
    _new_inputs(buf, 100)
    side = torch.cuda.Stream()  # warm-up off the capture stream: lazy buffers of the library and of torch exist afterwards
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(buf)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(buf)
    for rep in range(4):
        _new_inputs(buf, 200 + rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        scratch = torch.randn((1 << 20,), device=DEV).sum()  # eager work of the program's own between the replays
        want = step(buf)
        torch.cuda.synchronize()
        assert math.isfinite(float(scratch))
        for i, (g, w) in enumerate(zip(got, want)):
            assert torch.equal(g.nan_to_num(nan=-7.0), w.nan_to_num(nan=-7.0)), (rep, i)
        assert float(got[-1].float().abs().sum()) > 0 or float(buf["mask"].sum()) == 0


def test_single_pass_wide_row_first_launch_is_inside_the_capture():
    """Rows of 172032 bf16 logits take a build of the single-pass kernel that keeps part of the row in LDS and needs
    more dynamic LDS than a kernel gets by default.  `trlk_init` allows it beforehand, so the first launch of that
    build may sit inside a capture: no warm-up launch here."""
    from trl_amd import _lib, ops

    b, t, v = 2, 5, 172032
    assert v * 2 > 163840 * 2 and v <= ops.grpo_fused_max_vocab(torch.bfloat16)
    assert _lib.lib.trlk_init() == 0
    logits = torch.zeros((b, t, v), dtype=torch.bfloat16, device=DEV)
    ids = torch.zeros((b, t), dtype=torch.int64, device=DEV)
    mask = torch.ones((b, t), device=DEV)
    adv = torch.zeros((b,), device=DEV)
    row_scale = torch.full((b,), 1.0 / (b * t), device=DEV)

    def new_inputs(seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        logits.copy_((2.0 * torch.randn((b, t, v), generator=g, device=DEV)).bfloat16())
        ids.copy_(torch.randint(0, v, (b, t), generator=g, device=DEV))
        adv.copy_(torch.randn((b,), generator=g, device=DEV))
        mask.copy_((torch.rand((b, t), generator=g, device=DEV) < 0.8).float())

    def step():
        return ops.grpo_fused_fwd_bwd(logits, ids, 1.0, 0, t, mask, adv, row_scale, None, None, None, None,
                                      _lib.TERM_CLIP, 0.2, 0.28, math.nan, 0.0, False, 1.0, 1.05)

    new_inputs(300)
    ops.check_device_errors()
    ops._error_flag(torch.device(DEV))  # (the word the kernels report bad indices in exists before the capture)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(3):
        new_inputs(301 + rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in captured]
        scratch = torch.randn((1 << 20,), device=DEV).sum()
        want = step()
        torch.cuda.synchronize()
        assert math.isfinite(float(scratch))
        for i, (g_, w_) in enumerate(zip(got, want)):
            assert torch.equal(g_.nan_to_num(nan=-7.0), w_.nan_to_num(nan=-7.0)), (rep, i)
        assert float(got[-1].float().abs().sum()) > 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_fused_head_graph_replays_equal_eager(dtype):
    """Forward with its softmax numerators kept, then both gradient products from them: every buffer between the two
    (the kept numerators, the scaled fp16 operand copies, the maxima behind their scales) is rewritten inside the
    graph."""
    from trl_amd import ops

    n, h, v = 300, 128, 1000  # two token tiles, four vocabulary tiles, both with remainders
    hidden = torch.zeros((n, h), dtype=dtype, device=DEV)
    weight = torch.zeros((v, h), dtype=dtype, device=DEV)
    targets = torch.zeros((n,), dtype=torch.int64, device=DEV)
    g_logp = torch.zeros((n,), device=DEV)

    def new_inputs(seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        hidden.copy_(torch.randn((n, h), generator=g, device=DEV).to(dtype))
        weight.copy_((0.1 * torch.randn((v, h), generator=g, device=DEV)).to(dtype))
        targets.copy_(torch.randint(0, v, (n,), generator=g, device=DEV))
        g_logp.copy_(torch.randn((n,), generator=g, device=DEV) * (torch.rand((n,), generator=g, device=DEV) < 0.7))

    def step():
        lp, ent, log_z, hit, kept = ops.fused_head_fwd(hidden, weight, targets, 0.8, 0.0, 1.0, None, True)
        d_hidden, d_weight, _ = ops.fused_head_bwd(hidden, weight, targets, 0.8, 0.0, 1.0, log_z, g_logp, 512, None, kept)
        return lp, ent, hit, d_hidden, d_weight

    new_inputs(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(4):
        new_inputs(10 + rep)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        scratch = torch.randn((1 << 20,), device=DEV).sum()
        want = step()
        torch.cuda.synchronize()
        assert math.isfinite(float(scratch))
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (rep, i)
        assert float(got[3].float().abs().sum()) > 0 and float(got[4].float().abs().sum()) > 0


def test_two_host_threads_on_their_own_streams():
    """The entry points keep no state between calls (workspaces and outputs belong to the caller), so two host
    threads, each on a stream of its own, can run the two-pass step, the single-pass kernel and the fused head at the
    same time: each thread's results equal the ones the same inputs gave when run alone."""
    import threading

    import trl_amd
    from trl_amd import ops

    def make(seed):
        buf = _buffers()
        _new_inputs(buf, seed)
        g = torch.Generator(device=DEV).manual_seed(seed)
        head = (torch.randn((300, 128), generator=g, device=DEV).bfloat16(),
                (0.1 * torch.randn((1000, 128), generator=g, device=DEV)).bfloat16(),
                torch.randint(0, 1000, (300,), generator=g, device=DEV), torch.randn((300,), generator=g, device=DEV))
        return buf, head

    def work(buf, head):
        h, w, tg, gl = head
        # (the two-pass step through the ordinary loss entry point: the one that allocates nothing shares one
        # scratch array per GPU between all its callers and is documented as not to be overlapped)
        leaf = buf["logits"].detach().clone().requires_grad_(True)
        lp2, ent2 = trl_amd.per_token_logps_and_entropies(leaf, buf["ids"], T, 0.9, True, False)
        loss, metrics = trl_amd.grpo_loss(lp2, buf["adv"], buf["mask"], entropies=ent2,
                                          old_per_token_logps=lp2.detach() + buf["old_noise"], loss_type="dapo",
                                          epsilon_low=0.2, epsilon_high=0.28, num_items_in_batch=buf["n_items"])
        loss.backward()
        out = [lp2.detach(), ent2.detach(), loss.detach(), metrics.detach(), leaf.grad]
        out += [t.clone() for t in _single_pass_step(buf)]
        lp, ent, log_z, hit, kept = ops.fused_head_fwd(h, w, tg, 0.8, 0.0, 1.0, None, True)
        out += [lp, ent, *ops.fused_head_bwd(h, w, tg, 0.8, 0.0, 1.0, log_z, gl, 512, None, kept)[:2]]
        return out

    problems = [make(31), make(32)]
    torch.cuda.synchronize()
    alone = [work(*p) for p in problems]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def run(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(10):
                    results[i] = work(*problems[i])
            stream.synchronize()
        except Exception as exc:  # surfaced below, in the main thread
            errors.append(exc)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for i in range(2):
        for j, (a, b) in enumerate(zip(results[i], alone[i])):
            assert torch.equal(a.nan_to_num(nan=-7.0), b.nan_to_num(nan=-7.0)), (i, j)
