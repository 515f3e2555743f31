"""The entry point that allocates nothing (raven_qkv_attention_decode_static) against raven_qkv_attention_decode, through
the C ABI: the same bits in the output and in the appended cache rows, on two calls in a row, the second with a smaller
input (fewer sequences, a shorter cache, so that stale partial results of the first call lie behind the second's)."""

import pytest
import torch

from oracle import raven_oracle as O
from test_gpu_kernels import check, rnd

pytestmark = pytest.mark.gpu


def _case(pkg, B, T, nh, hd, dt, seed):
    h = nh * hd
    qkv = rnd((B, 3 * h), dt, seed).cuda()
    bias = rnd((2, nh, hd), dt, seed + 1, 0.1).cuda()
    table = O.rope_table(hd, T + 8, 50000.0)
    freqs = table.reshape(T + 8, hd // 2, 2).contiguous().cuda()
    k, v = rnd((2, B, nh, T + 1, hd), dt, seed + 2), rnd((2, B, nh, T + 1, hd), dt, seed + 3)
    return qkv, bias, freqs, k, v


@pytest.mark.parametrize("dt,nh,hd", [(torch.bfloat16, 55, 96), (torch.float32, 4, 64)])
def test_static_scratch_decode_attention_equals_workspace_version(pkg, tuned, dt, nh, hd):
    lib = pkg.hip.load()
    assert lib.raven_qkv_attention_decode_static_scratch_bytes() >= lib.raven_decode_attention_workspace_bytes(18, 55, 128)
    for call, (B, T) in enumerate([(3, 2100), (1, 700)]):  # both launches are split over positions by the library's rule
        qkv, bias, freqs, k, v = _case(pkg, B, T, nh, hd, dt, 40 + call)
        ka, va, kb, vb = k.cuda(), v.cuda(), k.cuda(), v.cuda()
        ws = pkg.hip.attention_workspace(B, nh, hd, "cuda")
        assert ws is not None
        want = pkg.hip.qkv_attention_decode(qkv, bias, freqs, pkg.hip.make_cache(ka, va), 1, B, T, nh, hd, workspace=ws)
        out = torch.empty(B, nh * hd, dtype=dt, device="cuda")
        got = pkg.hip.qkv_attention_decode_static(qkv, bias, freqs, pkg.hip.make_cache(kb, vb), 1, B, T, nh, hd, out=out)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"call {call}: output"
        assert torch.equal(ka, kb) and torch.equal(va, vb), f"call {call}: appended cache rows"
        if dt == torch.float32:
            # that the launch was split, seen from outside: one workgroup per (head, row) adds in another order
            tuned(attn_nosplit_pairs=1)
            kc, vc = k.cuda(), v.cuda()
            unsplit = pkg.hip.qkv_attention_decode(qkv, bias, freqs, pkg.hip.make_cache(kc, vc), 1, B, T, nh, hd, workspace=ws)
            tuned(attn_nosplit_pairs=165)
            assert not torch.equal(unsplit, want), f"call {call}: the launch under test was not split"
            check(unsplit, want, dt, f"call {call}: unsplit against split")
        # and both equal the oracle's attention over the T cached positions plus the new one
        h = nh * hd
        q_, k_, v_ = (t.view(B, 1, nh, hd) for t in qkv.cpu().split([h, h, h], dim=1))
        b_ = bias.cpu()
        q_, k_ = (q_ + b_[0]).to(dt), (k_ + b_[1]).to(dt)
        tab = O.rope_table(hd, T + 8, 50000.0)
        rq, rk = O.apply_rope(q_, k_, tab[:, T:T + 1])
        K = torch.cat([k[1, :, :, :T], rk.transpose(1, 2)], dim=2)
        V = torch.cat([v[1, :, :, :T], v_.transpose(1, 2)], dim=2)
        check(got, O.sdpa(rq.transpose(1, 2), K, V).transpose(1, 2).reshape(B, h), dt, f"call {call}: against the oracle")
    # with the device-side position (a replayed graph's form) the same again, and a launch that is never split
    qkv, bias, freqs, k, v = _case(pkg, 32, 300, nh, hd, dt, 60)
    ka, kb, va, vb = k.cuda(), k.cuda(), v.cuda(), v.cuda()
    pos_dev = torch.tensor([300], dtype=torch.int32, device="cuda")
    want = pkg.hip.qkv_attention_decode(qkv, bias, freqs, pkg.hip.make_cache(ka, va), 0, 32, 300, nh, hd, pos_dev=pos_dev,
                                        workspace=pkg.hip.attention_workspace(32, nh, hd, "cuda"))
    got = pkg.hip.qkv_attention_decode_static(qkv, bias, freqs, pkg.hip.make_cache(kb, vb), 0, 32, 300, nh, hd, pos_dev=pos_dev)
    assert torch.equal(got, want) and torch.equal(ka, kb)


def test_static_scratch_entry_allocates_nothing_and_replays_from_a_captured_graph(pkg):
    """What the entry point is for: after one eager call on the device (which looks the array's address up), a call
    leaves the allocator's counters where they were, and the call can be captured into a HIP graph -- position on the
    device, output buffer given -- and replayed: every replay gives the bits of the version with a workspace at that
    position, with eager work and synchronisations of the program between the replays."""
    dt, nh, hd, B, T = torch.bfloat16, 55, 96, 2, 1800   # long enough for the launch to be split
    qkv, bias, freqs, k, v = _case(pkg, B, T, nh, hd, dt, 70)
    ka, va, kb, vb = k.cuda(), v.cuda(), k.cuda(), v.cuda()
    ca, cb = pkg.hip.make_cache(ka, va), pkg.hip.make_cache(kb, vb)
    pos_dev = torch.tensor([T - 3], dtype=torch.int32, device="cuda")
    out = torch.empty(B, nh * hd, dtype=dt, device="cuda")
    ws = pkg.hip.attention_workspace(B, nh, hd, "cuda")
    pkg.hip.qkv_attention_decode_static(qkv, bias, freqs, cb, 1, B, T, nh, hd, pos_dev=pos_dev, out=out)   # the warm call
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"])
    pkg.hip.qkv_attention_decode_static(qkv, bias, freqs, cb, 1, B, T, nh, hd, pos_dev=pos_dev, out=out)
    torch.cuda.synchronize()
    assert before == (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pkg.hip.qkv_attention_decode_static(qkv, bias, freqs, cb, 1, B, T, nh, hd, pos_dev=pos_dev, out=out)
    for step in range(3):   # positions T - 3, T - 2, T - 1: the same graph, the position read from the device
        out.zero_()
        graph.replay()
        want = pkg.hip.qkv_attention_decode(qkv, bias, freqs, ca, 1, B, T, nh, hd, pos_dev=pos_dev, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {step}"
        assert torch.equal(ka, kb) and torch.equal(va, vb), f"replay {step}: appended rows"
        busy = (qkv.float() * 0.5 + 0.25).sum().item()   # eager work and a synchronisation between the replays
        assert busy == busy
        pkg.hip.advance_pos(pos_dev, 1)
