"""Pins of oracle/moe_scatter_gather.py: the reference's own test constructions (tests/kernels/test_scatter_gather.py)
run against the oracle, plus properties that fix what those leave open (order, bijection, untouched padding)."""
import random

import torch

import helpers
from oracle import moe_scatter_gather as sg


def reference_test_routing(seed, tokens=7, topk=8, experts=(6, 7, 8), picks=4, dtype=torch.int32):
    """The routing tables of tests/kernels/test_scatter_gather.py:27-34: `picks` random slots per token get a random
    expert of `experts` and a weight k / 10, the rest stay -1 / 0."""
    rng = random.Random(seed)
    ids = torch.full((tokens, topk), -1, dtype=dtype)
    w = torch.zeros(tokens, topk)
    for i in range(tokens):
        for _ in range(picks):
            idx = rng.randint(0, topk - 1)
            ids[i, idx] = rng.randint(experts[0], experts[-1])
            w[i, idx] = rng.randint(0, 10) / 10.0
    return ids, w


def scatter_case(seed, tokens=7, hidden=4096, E=32, per_expert=128, experts=(6, 7, 8), index_dtype=torch.int32):
    g = helpers.gen(seed)
    counts = [0] * E
    for e in experts:
        counts[e] = per_expert
    all_tokens = sum(counts)
    x = torch.randn(tokens, hidden, generator=g).to(torch.float8_e4m3fn)
    xs = torch.randn(tokens, hidden // 128, generator=g)
    ids, w = reference_test_routing(seed, tokens, 8, experts, dtype=index_dtype)
    return dict(x=x, xs=xs, ids=ids, w=w, counts=torch.tensor(counts, dtype=torch.int32), all_tokens=all_tokens, E=E)


def run_scatter(c, fill=0x33):
    out = torch.full((c['all_tokens'], c['x'].shape[1]), fill, dtype=torch.uint8).view(torch.float8_e4m3fn)
    out_s = torch.full((c['all_tokens'], c['xs'].shape[1]), -5.0)
    m_indices = torch.full((c['all_tokens'], ), -9, dtype=torch.int32)
    out_idx = torch.full_like(c['ids'], -1)
    start = torch.zeros(c['E'], dtype=torch.int64)
    sg.ep_scatter_ref(c['x'], c['xs'], c['ids'], c['counts'], start, out, out_s, m_indices, out_idx)
    return out, out_s, m_indices, out_idx, start


def test_scatter_reference_test_construction():
    # tests/kernels/test_scatter_gather.py:10-76 with the oracle in place of ep_scatter
    for seed in range(5):
        c = scatter_case(seed)
        out, out_s, m_indices, out_idx, _ = run_scatter(c)
        m_ref = torch.repeat_interleave(torch.arange(c['E'], dtype=torch.int32), c['counts'].long())
        assert torch.equal(m_indices, m_ref)
        out_ref = torch.full_like(out.view(torch.uint8), 0x33)
        out_s_ref = torch.full_like(out_s, -5.0)
        for i in range(c['ids'].shape[0]):
            for j in range(c['ids'].shape[1]):
                if c['ids'][i, j] >= 0:
                    dst = int(out_idx[i, j])
                    out_ref[dst] = c['x'].view(torch.uint8)[i]
                    out_s_ref[dst] = c['xs'][i]
        assert torch.equal(out.view(torch.uint8), out_ref) and torch.equal(out_s, out_s_ref)


def test_scatter_order_bijection_and_final_counters():
    c = scatter_case(11, tokens=40, hidden=256, E=8, per_expert=128, experts=(1, 2, 3, 4, 5))
    out, out_s, m_indices, out_idx, start = run_scatter(c)
    ids = c['ids']
    excl = torch.cumsum(c['counts'].long(), 0) - c['counts'].long()
    for e in range(c['E']):
        where = [(t, j) for t in range(ids.shape[0]) for j in range(ids.shape[1]) if int(ids[t, j]) == e]
        got = [int(out_idx[t, j]) for t, j in where]
        # token-major, slot-minor order onto consecutive rows from the expert's start
        assert got == list(range(int(excl[e]), int(excl[e]) + len(where)))
        assert int(start[e]) == int(excl[e]) + len(where)
    assert (out_idx[ids < 0] == -1).all()  # slots without an expert keep their content
    used = out_idx[ids >= 0]
    mask = torch.ones(c['all_tokens'], dtype=torch.bool)
    mask[used.long()] = False
    assert (out.view(torch.uint8)[mask] == 0x33).all() and (out_s[mask] == -5).all()  # padding rows untouched


def test_scatter_skips_ids_outside_the_expert_table():
    c = scatter_case(3, tokens=6, hidden=128, E=4, per_expert=128, experts=(1, 2))
    c['ids'][0, 0] = 9
    out, out_s, m_indices, out_idx, start = run_scatter(c)
    assert out_idx[0, 0] == -1


def test_gather_reference_test_construction_and_dense_formulation():
    for seed in range(4):
        g = helpers.gen(100 + seed)
        T, H, all_tokens = 7, 1024, 384
        ids, w = reference_test_routing(seed, T, 8)
        index = torch.randint(0, all_tokens, (T, 8), generator=g, dtype=torch.int32)
        inp = torch.randn(all_tokens, H, generator=g).to(torch.bfloat16)
        out = torch.full((T, H), 7.0, dtype=torch.bfloat16)
        sg.ep_gather_ref(inp, ids, w, index, out)
        # the accumulation loop of tests/kernels/test_scatter_gather.py:101-105 in fp32 (the reference test keeps its
        # sum in bf16 because its input is all zeros; fp32 is what the kernel it tests does, fused_moe_v3.py:178-186)
        ref = torch.zeros(T, H)
        for i in range(T):
            for j in range(8):
                if ids[i, j] >= 0:
                    ref[i] += inp[int(index[i, j])].float() * w[i, j]
        assert (out.float() - ref).abs().max() <= 2**-7 * ref.abs().max()
        # independent formulation: a dense [T, all_tokens] weight matrix times the input, in fp64
        dense = torch.zeros(T, all_tokens, dtype=torch.float64)
        for i in range(T):
            for j in range(8):
                if ids[i, j] >= 0:
                    dense[i, int(index[i, j])] += float(w[i, j])
        ref2 = (dense @ inp.double())
        assert ((out.double() - ref2).abs() <= ref2.abs() * 2**-8 + 1e-6).all()
        none = (ids < 0).all(dim=1)
        assert (out[none] == 0).all()


def test_scale_relayout_matches_transpose():
    g = helpers.gen(1)
    for m, k in ((1, 1), (7, 56), (130, 16), (128, 3)):
        s = torch.randn(m, k, generator=g)
        out = sg.tma_align_input_scale_ref(s)
        assert tuple(out.shape) == (m, k) and out.stride() == (1, (m + 3) // 4 * 4)
        assert torch.equal(out, s)
        assert torch.equal(out.t()[:, :m].contiguous(), s.t().contiguous())
