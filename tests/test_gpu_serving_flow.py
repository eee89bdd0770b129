"""A small serving loop end to end on the GPU: scheduler state -> PagedMetadataBuilder ->
TTAttentionBackendImpl.forward, for chunked prefill of requests of ragged length followed
by batched decode steps in a padded row bucket.  Each produced row is checked against
textbook fp32 causal attention over that request's whole K/V history held on the host (which
is what the reference's composition of fill / update / chunked / decode operators must
equal, attention.py:273-668 with metadata from model_runner.py:1722-2016), and the cache
contents are checked bit-exactly against the history at the end."""

import numpy as np
import pytest
import torch

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu

HQ, HKV, D, BS = 16, 4, 128, 32
WIDTH, BUDGET = 16, 128  # blocks per request, tokens per step


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def _expected(q_rows, hist_k, hist_v, first_pos):
    """q_rows [n, HQ, D] are the tokens at positions first_pos..first_pos+n-1 of a request
    whose K/V history is hist_* [len, HKV, D]."""
    n = q_rows.shape[0]
    total = first_pos + n
    group = HQ // HKV
    k = hist_k[:total].float().repeat_interleave(group, dim=1)  # [total, HQ, D]
    v = hist_v[:total].float().repeat_interleave(group, dim=1)
    scores = torch.einsum("nhd,thd->hnt", q_rows.float(), k) * D**-0.5
    key_pos = torch.arange(total).view(1, 1, total)
    query_pos = (first_pos + torch.arange(n)).view(1, n, 1)
    scores = scores.masked_fill(key_pos > query_pos, float("-inf"))
    return torch.einsum("hnt,thd->nhd", torch.softmax(scores, dim=-1), v)  # [n, HQ, D] fp32


@pytest.mark.parametrize("spec_rows", [False, True])
def test_chunked_prefill_then_batched_decode(spec_rows):
    from tt_xla_amd import TTAttentionBackendImpl
    from tt_xla_amd.metadata import PagedMetadataBuilder

    gen = torch.Generator().manual_seed(11 + spec_rows)
    prompt = [200, 205, 77, 333]
    reqs = len(prompt)
    nb = reqs * WIDTH + 1  # block 0 is the null block
    block_table = (torch.randperm(nb - 1, generator=gen) + 1).view(reqs, WIDTH).numpy().astype(np.int32)
    kv = [torch.zeros(nb, HKV, BS, D, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    impl = TTAttentionBackendImpl(HQ, D, D**-0.5, HKV, None, None, "auto")
    builder = PagedMetadataBuilder(BS, WIDTH, BUDGET, device="cuda", spec_prefix_rows=spec_rows)

    decode_steps = 6 if not spec_rows else 3
    total_len = [p + decode_steps * (1 if not spec_rows else 3) for p in prompt]
    assert max(total_len) <= WIDTH * BS
    # Every token's q/k/v for the whole life of each request, fixed up front.
    q_all = [_bf(gen, n, HQ, D) for n in total_len]
    k_all = [_bf(gen, n, HKV, D) for n in total_len]
    v_all = [_bf(gen, n, HKV, D) for n in total_len]
    computed = np.zeros(reqs, dtype=np.int64)
    worst = 0.0

    def run_pass(rows_of, sched, target):
        """rows_of: request index of each pass row; sched: tokens per pass row."""
        nonlocal worst
        comp = computed[rows_of]
        plan = builder.prepare(block_table[rows_of], comp, np.asarray(sched), target_num_reqs=target)
        md, L = plan.metadata, plan.padded_tokens
        q = torch.zeros(target, L, HQ, D, dtype=torch.bfloat16)
        k = torch.zeros(target, L, HKV, D, dtype=torch.bfloat16)
        v = torch.zeros(target, L, HKV, D, dtype=torch.bfloat16)
        for r, (req, n) in enumerate(zip(rows_of, sched)):
            first = int(comp[r]) - int(plan.row_lead[r])
            n_row = n + int(plan.row_lead[r])
            assert plan.positions[r, :n_row].tolist() == list(range(first, first + n_row))
            q[r, :n_row] = q_all[req][first : first + n_row]
            k[r, :n_row] = k_all[req][first : first + n_row]
            v[r, :n_row] = v_all[req][first : first + n_row]
        out = torch.empty(target * L, HQ * D, dtype=torch.bfloat16, device="cuda")
        impl.forward(None, q.view(target * L, HQ * D).cuda(), k.view(target * L, HKV * D).cuda(),
                     v.view(target * L, HKV * D).cuda(), kv, md, output=out)
        out = out.cpu().view(target, L, HQ, D)
        for r, (req, n) in enumerate(zip(rows_of, sched)):
            first = int(comp[r]) - int(plan.row_lead[r])
            n_row = n + int(plan.row_lead[r])
            want = _expected(q_all[req][first : first + n_row], k_all[req], v_all[req], first)
            got = out[r, :n_row]
            worst = max(worst, (got.float() - want.float()).abs().max().item())
            torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)
            computed[req] += n

    # Chunked prefill, one request per pass (rows at different stages cannot share a pass).
    for req in range(reqs):
        while computed[req] < prompt[req]:
            n = int(min(BUDGET, prompt[req] - computed[req]))
            run_pass([req], [n], target=1)
    assert computed.tolist() == prompt

    if not spec_rows:
        # Batched single-token decode in a padded bucket of 8 rows.
        for _ in range(decode_steps):
            run_pass(list(range(reqs)), [1] * reqs, target=8)
    else:
        # Multi-token (speculative) decode rows start mid-block: each pass is trimmed to
        # the run of requests sharing one block boundary and re-feeds row_lead tokens.
        for _ in range(decode_steps):
            pending = list(range(reqs))
            while pending:
                run = builder.trim_pass(computed[pending], np.full(len(pending), 3))
                run_pass(pending[:run], [3] * run, target=4)
                pending = pending[run:]
    assert computed.tolist() == total_len

    # Cache contents: every position of every request holds exactly the token's K / V.
    table = torch.from_numpy(block_table)
    kc, vc = kv[0].cpu(), kv[1].cpu()
    for req in range(reqs):
        n = total_len[req]
        pos = torch.arange(n)
        blocks = table[req, pos // BS].long()
        got_k = kc[blocks, :, pos % BS]  # [n, HKV, D]
        got_v = vc[blocks, :, pos % BS]
        assert torch.equal(got_k, k_all[req]) and torch.equal(got_v, v_all[req])
    print(f"serving flow max-abs error {worst:.3e}")
