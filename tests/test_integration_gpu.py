"""Operator-level integration on an MI355X: graph capture, side streams, the registry / executor wiring."""
import pytest
import torch

from benchmarks.workloads import cfg5_sampling, spike_block
from oracle import exact, logprob_ref

pytestmark = pytest.mark.gpu


def test_hip_graph_replays_match_eager(sampler):
    """The kernels hold no host-side state and record no memset nodes: a captured logprob + sampling +
    fused lm_head sequence must replay to the eager result every time."""
    logits, ids = spike_block(256, 32000, seed=3, block=0, device="cuda")
    slog, u = cfg5_sampling(32, device="cuda", vocab=32000)
    g = torch.Generator(device="cuda").manual_seed(1)
    hidden = torch.randn(300, 256, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(5000, 256, generator=g, device="cuda") * 0.1).bfloat16()
    hid = torch.randint(0, 5000, (300,), generator=g, device="cuda")
    eager = (sampler.compute_logp(logits, ids), sampler.sample(slog, top_k=50, top_p=0.9, temperature=0.7, uniforms=u),
             sampler.fused_linear_logp(hidden, weight, hid),
             sampler.sample(slog, top_p=0.9, temperature=0.7, uniforms=u),      # dense-histogram path (157 KB of LDS)
             sampler.sample(slog, uniforms=u))                                   # no filter
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lp = sampler.compute_logp(logits, ids)
        tok = sampler.sample(slog, top_k=50, top_p=0.9, temperature=0.7, uniforms=u)
        fl = sampler.fused_linear_logp(hidden, weight, hid)
        tok_p = sampler.sample(slog, top_p=0.9, temperature=0.7, uniforms=u)
        tok_all = sampler.sample(slog, uniforms=u)
    for replay in range(3):
        with torch.inference_mode():  # the operators return inference tensors, as the reference's do
            lp.zero_(); tok.zero_(); fl.zero_(); tok_p.zero_(); tok_all.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(lp, eager[0]) and torch.equal(tok, eager[1]) and torch.equal(fl, eager[2]), replay
        assert torch.equal(tok_p, eager[3]) and torch.equal(tok_all, eager[4]), replay
        assert torch.equal(tok_p.cpu(), exact.sample(slog.cpu(), 0.7, None, 0.9, u.cpu()))
        # eager work between replays
        assert torch.equal(sampler.compute_logp(logits, ids), eager[0])


def test_side_stream(sampler):
    logits, ids = spike_block(512, 32000, seed=4, block=0, device="cuda")
    want = sampler.compute_logp(logits, ids)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        got = sampler.compute_logp(logits, ids)
    stream.synchronize()
    assert torch.equal(got, want)


def test_registry_resolves_to_the_hip_operators():
    from rl_engine.executors.rollout import RolloutExecutor
    from rl_engine.kernels.registry import kernel_registry

    logits, u = cfg5_sampling(16, device="cuda", vocab=32000)
    executor = RolloutExecutor({"top_k": 50, "top_p": 0.9, "temperature": 0.7})
    ids, logp = executor.step(logits, uniforms=u)
    assert torch.equal(ids.cpu(), exact.sample(logits.cpu(), 0.7, 50, 0.9, u.cpu()))
    want = logprob_ref.logprob_ref(logits.cpu(), ids.cpu())
    assert (logp.cpu() - want).abs().max().item() <= 1e-4
    assert kernel_registry.resolve("fused_lm_head_logp").__name__ == "fused_linear_logp"


def test_generate_loop_matches_stepwise_oracle():
    """A toy next-token model (logits = table[last id]) rolled out for 6 steps: every step's ids equal the exact
    oracle's on the same logits and uniforms, logprobs are those of the unfiltered rows, rows that hit the
    end-of-sequence id stay there."""
    from rl_engine.executors.rollout import RolloutExecutor

    gen = torch.Generator().manual_seed(77)
    vocab, batch, steps, eos = 4096, 8, 6, 5
    table = (torch.randn(vocab, vocab, generator=gen) * 3.0).bfloat16()
    table[:, eos] += 4.0                                     # make the end id likely enough to show up
    prompt = torch.randint(0, vocab, (batch, 3), generator=gen)
    u = torch.rand(steps, batch, generator=gen)
    table_gpu = table.cuda()
    executor = RolloutExecutor({"top_k": 20, "top_p": 0.95, "temperature": 0.8})
    ids, logp = executor.generate(lambda seq: table_gpu[seq[:, -1]], prompt.cuda(), steps, uniforms=u.cuda(), eos_id=eos)
    assert ids.shape == (batch, 3 + steps) and torch.equal(ids[:, :3].cpu(), prompt)

    cur, done = prompt[:, -1].clone(), torch.zeros(batch, dtype=torch.bool)
    for s in range(steps):
        rows = table[cur]
        tok = exact.sample(rows, 0.8, 20, 0.95, u[s])
        lp = logprob_ref.logprob_ref(rows, tok)
        tok = torch.where(done, torch.full_like(tok, eos), tok)
        lp = torch.where(done, torch.zeros_like(lp), lp)
        done |= tok == eos
        assert torch.equal(ids[:, 3 + s].cpu(), tok), s
        assert (logp[:, s].cpu() - lp).abs().max().item() <= 1e-4
        cur = tok
    assert done.any()


def test_large_batch_sampling_replayed_from_a_hip_graph(sampler):
    """A batch of more rows than the device has CUs runs the short top-k route with two rows resident per CU: captured and
    replayed, ids and policy log-probabilities equal the eager call's and the oracle's ids."""
    from oracle import exact

    slog, u = cfg5_sampling(600, device="cuda", vocab=32000)
    eager = sampler.sample(slog, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ids, pol = sampler.sample(slog, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
    for _ in range(3):
        with torch.inference_mode():
            ids.zero_(); pol.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ids, eager[0]) and torch.equal(pol.view(torch.int32), eager[1].view(torch.int32))
        junk = torch.randn(1 << 18, device="cuda").sum().item()          # eager work between replays
        assert junk == junk
    assert torch.equal(ids.cpu(), exact.sample(slog.cpu(), 0.7, 50, 0.9, u.cpu()))


def test_decode_step_replayed_from_a_hip_graph(sampler):
    """GraphedDecodeStep records sample + compute_logp once and replays them: every replay - with the program's own
    eager work and synchronisations between them - must give the eager operators' results bit for bit, and those
    of the CPU oracles."""
    from oracle import exact, logprob_ref
    from rl_engine.kernels.graphs import GraphedDecodeStep

    batch, vocab = 24, 32000
    step = GraphedDecodeStep(sampler, batch, vocab, top_k=50, top_p=0.9, temperature=0.7)
    g = torch.Generator().manual_seed(71)
    for it in range(4):
        logits = (torch.randn(batch, vocab, generator=g) * 3).bfloat16()
        u = torch.rand(batch, generator=g)
        if it % 2 == 0:
            ids, logp = step(logits.cuda(), u.cuda())
        else:                                          # the caller writes the inputs itself
            step.logits.copy_(logits.cuda())
            step.uniforms.copy_(u.cuda())
            ids, logp = step()
        got_ids, got_logp = ids.clone(), logp.clone()
        torch.cuda.synchronize()
        eager_ids, eager_logp = sampler.sample(logits.cuda(), top_k=50, top_p=0.9, temperature=0.7, uniforms=u.cuda(),
                                               return_policy_logprob=True)
        assert (eager_logp - sampler.compute_logp(logits.cuda(), eager_ids)).abs().max().item() <= 1e-5
        junk = torch.randn(1 << 20, device="cuda").sum().item()          # eager work and a sync between replays
        assert junk == junk
        assert torch.equal(got_ids, eager_ids) and torch.equal(got_logp, eager_logp)
        assert torch.equal(got_ids.cpu(), exact.sample(logits, 0.7, 50, 0.9, u))
        assert (got_logp.cpu() - logprob_ref.logprob_ref(logits, got_ids.cpu())).abs().max().item() <= 1e-4


def test_policy_logprob_from_the_sampling_call(sampler):
    """sample(..., return_policy_logprob=True): the drawn token's log-probability under the unfiltered softmax comes
    out of the sampling kernel itself.  Same ids as without it; the value is compute_logp's to 1e-5 (another fixed
    summation order) and the oracle's to 1e-4, on every route (short top-k, block-wide top-k, dense histogram, radix,
    fp32 rows, unaligned rows, a masked vocabulary), alone and together with the filtered log-probability."""
    from oracle import logprob_ref
    from rl_engine.kernels import _hip

    g = torch.Generator().manual_seed(81)
    cases = [dict(top_k=50, top_p=0.9, temperature=0.7), dict(top_k=200, temperature=1.3), dict(top_k=700, top_p=0.95),
             dict(top_p=0.9, temperature=0.7), dict(top_p=0.9), dict(), dict(top_k=3000, top_p=0.9)]
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        host = (torch.randn(40, 9000, generator=g) * 3).to(dtype)
        host[5, 4000:] = float("-inf")                                   # masked tail
        host[6, ::3] = 7.0                                               # 3,000-way tie at the top
        logits = host.cuda()
        u = torch.rand(40, generator=g).cuda()
        for kw in cases:
            for flags in (0, _hip.SAMPLE_FLAG_BLOCK_WIDE_TOPK, _hip.SAMPLE_FLAG_GENERAL_PATH):
                ids, policy = sampler.sample(logits, uniforms=u, return_policy_logprob=True, route_flags=flags, **kw)
                assert torch.equal(ids, sampler.sample(logits, uniforms=u, **kw)), (dtype, kw, flags)
                assert (policy - sampler.compute_logp(logits, ids)).abs().max().item() <= 1e-5, (dtype, kw, flags)
                assert (policy.cpu() - logprob_ref.logprob_ref(host, ids.cpu())).abs().max().item() <= 1e-4
        ids2, lp, policy2 = sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_logprob=True,
                                           return_policy_logprob=True)
        ids1, policy1 = sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
        assert torch.equal(ids2, ids1) and torch.equal(policy2, policy1) and (lp <= 0).all()
        # without a temperature the filters only remove mass: the drawn token's filtered probability is at least its policy one
        _, lp1, pol1 = sampler.sample(logits, top_k=50, top_p=0.9, uniforms=u, return_logprob=True, return_policy_logprob=True)
        assert (lp1 >= pol1 - 1e-5).all()
        # an unaligned view (scalar loads) and a batch split give the same values
        view = logits[:, 3:8000]
        a_ids, a_pol = sampler.sample(view, top_k=50, uniforms=u, return_policy_logprob=True)
        assert (a_pol - sampler.compute_logp(view, a_ids)).abs().max().item() <= 1e-5
        parts = [sampler.sample(logits[s0:s0 + 10], top_k=50, top_p=0.9, temperature=0.7, uniforms=u[s0:s0 + 10],
                                return_policy_logprob=True)[1] for s0 in range(0, 40, 10)]
        assert torch.equal(torch.cat(parts), policy1)
    e_ids, e_pol = sampler.sample(torch.empty(0, 100, dtype=torch.bfloat16, device="cuda"), return_policy_logprob=True)
    assert e_ids.numel() == 0 and e_pol.numel() == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_policy_logprob_on_rows_that_start_with_masked_entries(sampler, dtype):
    """The log-sum-exp that the sampling kernel takes along uses the same floor-started running maximum as the logprob
    kernel: a masked prefix (a lane's first entries are all -inf), every other entry masked, a single finite entry at
    the end of the row.  At the headline row length, on every route, against compute_logp (1e-5) and the oracle (1e-4)."""
    from oracle import logprob_ref
    from rl_engine.kernels import _hip

    g = torch.Generator().manual_seed(83)
    host = (torch.randn(10, 128256, generator=g) * 3).to(dtype)
    host[0, :70000] = float("-inf")
    host[1, :1000] = float("-inf")
    host[2, 1::2] = float("-inf")
    host[3, :] = float("-inf")
    host[3, 128255] = 1.0
    host[4, :128000] = float("-inf")                                     # fewer finite entries than top_k = 500
    logits, u = host.cuda(), torch.rand(10, generator=g).cuda()
    for kw in (dict(top_k=50, top_p=0.9, temperature=0.7), dict(top_k=200), dict(top_k=500, top_p=0.95), dict(top_p=0.9),
               dict()):
        for flags in (0, _hip.SAMPLE_FLAG_BLOCK_WIDE_TOPK, _hip.SAMPLE_FLAG_GENERAL_PATH):
            ids, policy = sampler.sample(logits, uniforms=u, return_policy_logprob=True, route_flags=flags, **kw)
            assert torch.equal(ids.cpu(), exact.sample(host, kw.get("temperature", 1.0), kw.get("top_k"), kw.get("top_p"), u.cpu()))
            assert torch.isfinite(policy).all(), (dtype, kw, flags)
            assert (policy - sampler.compute_logp(logits, ids)).abs().max().item() <= 1e-5, (dtype, kw, flags)
            assert (policy.cpu() - logprob_ref.logprob_ref(host, ids.cpu())).abs().max().item() <= 1e-4
            assert ids[3].item() == 128255 and abs(policy[3].item()) <= 1e-6


def test_policy_logprob_at_the_benchmark_shape_and_with_per_row_parameters(sampler):
    """bf16 [256, 128256] as the sampling benchmark draws it: ids against the oracle, the policy log-probability against
    compute_logp and the oracle; then one call with per-row top_k / top_p / temperature tensors (the kernel variant
    with the dense-histogram LDS, whose routes pass over the row once more for the log-sum-exp) and a ragged fp32 row
    length that takes several tracking rounds."""
    from benchmarks.workloads import cfg5_sampling
    from oracle import logprob_ref

    host, u = cfg5_sampling(256)
    logits, ug = host.cuda(), u.cuda()
    ids, policy = sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=ug, return_policy_logprob=True)
    assert torch.equal(ids.cpu(), exact.sample(host, 0.7, 50, 0.9, u))
    assert (policy - sampler.compute_logp(logits, ids)).abs().max().item() <= 1e-5
    assert (policy.cpu() - logprob_ref.logprob_ref(host, ids.cpu())).abs().max().item() <= 1e-4
    g = torch.Generator().manual_seed(84)
    k_rows = torch.randint(0, 3000, (256,), generator=g).to(torch.int32)          # 0 = off; beyond 1024: dense histogram
    k_rows[:32] = torch.randint(1, 64, (32,), generator=g).to(torch.int32)
    p_rows = torch.rand(256, generator=g) * 0.6 + 0.4
    p_rows[::7] = 1.0
    t_rows = torch.rand(256, generator=g) * 1.5 + 0.25
    ids2, policy2 = sampler.sample(logits, top_k=k_rows.cuda(), top_p=p_rows.cuda(), temperature=t_rows.cuda(),
                                   uniforms=ug, return_policy_logprob=True)
    want = exact.sample_rows(host, t_rows, k_rows, p_rows, u)[0]
    assert torch.equal(ids2.cpu(), want)
    assert (policy2 - sampler.compute_logp(logits, ids2)).abs().max().item() <= 1e-5
    assert (policy2.cpu() - logprob_ref.logprob_ref(host, ids2.cpu())).abs().max().item() <= 1e-4
    wide = (torch.randn(6, 300003, generator=g) * 3)                              # fp32, ragged, three tracking rounds
    wide[1, :150000] = float("-inf")
    uw = torch.rand(6, generator=g)
    ids3, policy3 = sampler.sample(wide.cuda(), top_k=40, top_p=0.9, temperature=0.8, uniforms=uw.cuda(),
                                   return_policy_logprob=True)
    assert torch.equal(ids3.cpu(), exact.sample(wide, 0.8, 40, 0.9, uw))
    assert (policy3.cpu() - logprob_ref.logprob_ref(wide, ids3.cpu())).abs().max().item() <= 1e-4


def test_captured_fused_linear_logp_owns_its_workspace(sampler):
    """A fused_linear_logp captured in a HIP graph takes its scratch from the graph's own memory, not from the backend's
    arena: replays on one stream run while eager calls (which lease the arena) run on another, and both results stay
    bit-equal to sequential calls.  The two inputs are sized so that their partial results would overlap in the arena."""
    def make(n, seed):
        g = torch.Generator(device="cuda").manual_seed(seed)
        return (torch.randn(n, 512, generator=g, device="cuda").bfloat16(),
                (torch.randn(30000, 512, generator=g, device="cuda") * 0.05).bfloat16(),
                torch.randint(0, 30000, (n,), generator=g, device="cuda"))

    a, b = make(2048, 41), make(1792, 42)
    want_a, want_b = sampler.fused_linear_logp(*a), sampler.fused_linear_logp(*b)
    torch.cuda.synchronize()
    arena_before = sampler.pool._last_use.get(0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got_a = sampler.fused_linear_logp(*a)
    assert sampler.pool._last_use.get(0) is arena_before          # the capture left no event behind in the pool
    side = torch.cuda.Stream()
    for _ in range(4):
        with torch.inference_mode():
            got_a.zero_()
        torch.cuda.synchronize()
        graph.replay()                                             # on the current stream
        with torch.cuda.stream(side):
            got_b = [sampler.fused_linear_logp(*b) for _ in range(3)]  # eager, arena, other stream, concurrently
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got_a, want_a)
        assert all(torch.equal(x, want_b) for x in got_b)
