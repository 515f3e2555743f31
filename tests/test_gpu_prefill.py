"""GPU parity at the prefill configuration (core prefill at the 3.5b shape: 4 sequences x 4096 tokens, bf16) and of the
tiled MFMA GEMM that serves every product with 33 or more token rows.

All calls go through the C ABI (pkg.hip wrappers).  Reference values: fp32 `F.linear` on the same operands for the
products (the library's GEMMs are row-independent, so a sample of rows is compared at full N), the CPU oracle's
`sdpa` per head for attention, and the oracle's SandwichBlock on a sample of rows of one sequence for the composed block
(attention needs all keys of that sequence, so its K / V rows are all computed by the oracle).
Bars: per kernel max-abs <= 2e-2 (times max(1, |ref|max)) and rel-L2 <= 1e-2; the composed block as in test_gpu_model.py."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import raven_oracle as O
from test_gpu_kernels import ULPS_COMPOSED, ULPS_RESIDUAL, ULPS_SWIGLU, check, close, rnd

pytestmark = pytest.mark.gpu

H, NH, HD, INTER = 5280, 55, 96, 17920


def _rows(M, n=48, seed=0):
    """Rows to compare: the first and last tile edges plus a random sample."""
    g = torch.Generator().manual_seed(seed)
    picks = [torch.arange(0, min(M, 8)), torch.arange(max(0, M - 8), M), torch.randint(0, M, (n,), generator=g)]
    for edge in (255, 256, 257, 4095, 4096, 8191, 8192):
        if edge < M:
            picks.append(torch.tensor([edge]))
    return torch.unique(torch.cat(picks))


def _gpu_randn(shape, seed, std=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * std).to(torch.bfloat16)


def _ref_rows(x, w, rows):
    """fp32 product of the sampled rows with the whole matrix (a plain PyTorch fp32 reference of nn.Linear)."""
    return F.linear(x[rows].float(), w.float())


# ----------------------------------------------------------------------------- the five products at M = 16384
@pytest.mark.parametrize("name", ["Wqkv", "attn.proj", "mlp.fc", "mlp.proj", "adapter", "lm_head"])
def test_tiled_gemm_nebel_shapes_m16384(pkg, name):
    """RMM:463, 493, 507-509, 776, 711 at 16384 token rows: the tiled kernel with each product's epilogue."""
    dt, M = torch.bfloat16, 16384
    rows = _rows(M).cuda()
    kw = {}
    if name == "Wqkv":
        x, w = _gpu_randn((M, H), 1), _gpu_randn((3 * H, H), 2, 0.02)
        got = pkg.hip.linear(x, w)
        want = _ref_rows(x, w, rows).to(dt)
    elif name == "attn.proj":
        x, w, res = _gpu_randn((M, H), 3), _gpu_randn((H, H), 4, 0.02), _gpu_randn((M, H), 5)
        got = pkg.hip.linear(x, w, residual=res)
        want = (_ref_rows(x, w, rows).to(dt).float() + res[rows].float()).to(dt)
        kw = dict(mag=_ref_rows(x, w, rows), ulps=ULPS_RESIDUAL)
    elif name == "mlp.fc":
        x, w = _gpu_randn((M, H), 6), _gpu_randn((2 * INTER, H), 7, 0.02)
        got = pkg.hip.linear(x, w, swiglu=True)
        z = _ref_rows(x, w, rows).to(dt).float()
        want = (F.silu(z[:, :INTER]).to(dt).float() * z[:, INTER:]).to(dt)
        wrong = (F.silu(z[:, INTER:]).to(dt).float() * z[:, :INTER]).to(dt)
        assert close(got[rows], wrong)[1] > 0.1, "the gate must be the first half of fc's output"
        kw = dict(ulps=ULPS_SWIGLU)
    elif name == "mlp.proj":
        x, w, res = _gpu_randn((M, INTER), 8), _gpu_randn((H, INTER), 9, 0.02), _gpu_randn((M, H), 10)
        got = pkg.hip.linear(x, w, residual=res)
        want = (_ref_rows(x, w, rows).to(dt).float() + res[rows].float()).to(dt)
        kw = dict(mag=_ref_rows(x, w, rows), ulps=ULPS_RESIDUAL)
    elif name == "adapter":
        x0, x1, w = _gpu_randn((M, H), 11), _gpu_randn((M, H), 12), _gpu_randn((H, 2 * H), 13, 0.02)
        got = pkg.hip.linear(x0, w, x1=x1)
        want = _ref_rows(torch.cat([x0[rows], x1[rows]], -1), w, torch.arange(rows.numel()).cuda()).to(dt)
        swapped = _ref_rows(torch.cat([x1[rows], x0[rows]], -1), w, torch.arange(rows.numel()).cuda()).to(dt)
        assert close(got[rows], swapped)[1] > 0.1, "the state is the first operand, the embedded input the second"
    else:  # lm_head: a quarter of the rows is enough for a 65536-wide output (float logits)
        M = 4096
        rows = _rows(M).cuda()
        x, w = _gpu_randn((M, H), 14), _gpu_randn((65536, H), 15, 0.02)
        got = pkg.hip.gemm(x, w, out_f32=True)
        assert got.dtype == torch.float32
        want = _ref_rows(x, w, rows).to(dt).float()
    check(got[rows], want, dt, f"{name} at {M} rows", **kw)
    assert torch.isfinite(got.float()).all()


@pytest.mark.parametrize("M", [33, 64, 65, 96, 128, 129, 160, 161])
def test_products_around_the_switch_between_skinny_passes_and_tiles(pkg, M):
    """33 to 161 token rows with the default dispatch: which kernel takes a product changes with the row count here
    (passes of the 32-row kernels up to 64 rows at K = 5280, 128 at 10560, 160 at 17920; 128 x 128 tiles beyond).  The five
    products of the 3.5b shape, each with its epilogue, on either side of every switch, against fp32 F.linear."""
    dt = torch.bfloat16
    x, e, res = _gpu_randn((M, H), 20 + M), _gpu_randn((M, H), 21 + M), _gpu_randn((M, H), 22 + M)
    g = _gpu_randn((M, INTER), 23 + M)
    rows = torch.arange(M).cuda()
    w = _gpu_randn((3 * H, H), 30, 0.02)
    check(pkg.hip.linear(x, w), _ref_rows(x, w, rows).to(dt), dt, f"Wqkv at {M} rows")
    w = _gpu_randn((H, H), 31, 0.02)
    p = _ref_rows(x, w, rows)
    check(pkg.hip.linear(x, w, residual=res), (p.to(dt).float() + res.float()).to(dt), dt, f"attn.proj at {M} rows", mag=p, ulps=ULPS_RESIDUAL)
    w = _gpu_randn((2 * INTER, H), 32, 0.02)
    z = _ref_rows(x, w, rows).to(dt).float()
    check(pkg.hip.linear(x, w, swiglu=True), (F.silu(z[:, :INTER]).to(dt).float() * z[:, INTER:]).to(dt), dt, f"mlp.fc at {M} rows",
          ulps=ULPS_SWIGLU)
    w = _gpu_randn((H, INTER), 33, 0.02)
    p = _ref_rows(g, w, rows)
    check(pkg.hip.linear(g, w, residual=res), (p.to(dt).float() + res.float()).to(dt), dt, f"mlp.proj at {M} rows", mag=p, ulps=ULPS_RESIDUAL)
    w = _gpu_randn((H, 2 * H), 34, 0.02)
    check(pkg.hip.linear(x, w, x1=e), _ref_rows(torch.cat([x, e], -1), w, rows).to(dt), dt, f"adapter at {M} rows")


@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(33, 64, 64), (64, 256, 256), (100, 264, 320), (257, 520, 96), (300, 5280, 5280), (513, 776, 1096), (700, 1032, 136)])
def test_tiled_gemm_edges_against_oracle(pkg, tuned, variant, M, N, K):
    """The three tile kernels (256 x 256 by four waves with an LDS ring, 128 x 128, 256 x 256 by eight waves with staging
    registers) on shapes with partial tiles in M and N, K that is not a multiple of the 64-wide step (down to one and
    two steps, fewer than the ring holds), every epilogue and the two-operand form, against the oracle's linear /
    SwiGLU / residual."""
    dt = torch.bfloat16
    tuned(gemm_tiled_variant=variant)
    x, w, res = rnd((M, K), dt, 500 + M), rnd((N, K), dt, 501 + N, 0.05), rnd((M, N), dt, 502)
    dev = lambda t: t.cuda()
    lin = lambda a, b: F.linear(a.float(), b.float())
    check(pkg.hip.linear(dev(x), dev(w)), lin(x, w).to(dt), dt, "plain")
    check(pkg.hip.linear(dev(x), dev(w), residual=dev(res)), lin(x, w).to(dt) + res, dt, "+ residual", mag=lin(x, w), ulps=ULPS_RESIDUAL)
    yf = pkg.hip.linear(dev(x), dev(w), out_f32=True)
    assert yf.dtype == torch.float32 and torch.equal(yf, pkg.hip.linear(dev(x), dev(w)).float())
    if N % 16 == 0:
        fc = rnd((2 * N, K), dt, 503, 0.05)
        z = lin(x, fc).to(dt)
        check(pkg.hip.linear(dev(x), dev(fc), swiglu=True), F.silu(z[:, :N]) * z[:, N:], dt, "SwiGLU", ulps=ULPS_SWIGLU)
    x1, w2 = rnd((M, K), dt, 504), rnd((N, 2 * K), dt, 505, 0.05)
    check(pkg.hip.linear(dev(x), dev(w2), x1=dev(x1)), lin(torch.cat([x, x1], -1), w2).to(dt), dt, "two operands")
    # against the oracle's own statement of the products (nn.Linear in bf16 on the CPU; small shapes only: it is slow)
    if M * N * K <= 2 * 10 ** 8:
        check(pkg.hip.linear(dev(x), dev(w)), O.linear(x, w), dt, "oracle linear")
    # the same call twice: the same bits; and the tile size does not change a bit either (one accumulation order)
    a = pkg.hip.linear(dev(x), dev(w))
    for other in {1, 2, 3} - {variant}:
        tuned(gemm_tiled_variant=other)
        assert torch.equal(a, pkg.hip.linear(dev(x), dev(w))), (variant, other)


@pytest.mark.parametrize("N", [16640, 16544])
def test_tiled_gemm_last_round_as_small_tiles_changes_no_bit(pkg, tuned, N):
    """4 x 65 tiles of 256 x 256 (4 x 130 under SwiGLU): the tiles of the last, nearly empty round (the last tile
    columns, whole or partly filled) are multiplied as 128 x 128 tiles by a second launch over that column range.  Same
    bits as one launch, for every epilogue, and right against the fp32 product on sampled columns of both ranges."""
    dt, M, K = torch.bfloat16, 1024, 192
    x, x1 = _gpu_randn((M, K), 600), _gpu_randn((M, K), 601)
    w, w2, res = _gpu_randn((N, K), 602, 0.05), _gpu_randn((N, 2 * K), 603, 0.05), _gpu_randn((M, N), 604)
    fc = _gpu_randn((2 * N, K), 605, 0.05)
    calls = {"plain": lambda: pkg.hip.linear(x, w), "+ residual": lambda: pkg.hip.linear(x, w, residual=res),
             "float": lambda: pkg.hip.linear(x, w, out_f32=True), "two operands": lambda: pkg.hip.linear(x, w2, x1=x1),
             "SwiGLU": lambda: pkg.hip.linear(x, fc, swiglu=True)}
    for name, call in calls.items():
        tuned(gemm_tiled_split_tail=1)
        split = call()
        tuned(gemm_tiled_split_tail=0)
        whole = call()
        assert torch.equal(split, whole), name
    cols = torch.tensor([0, 255, 256, 8191, 16383, 16384, 16385, 16511, 16512, N - 1]).cuda()
    tuned(gemm_tiled_split_tail=1)
    want = (x.float() @ w[cols].float().T).to(dt).float() + res[:, cols].float()
    check(pkg.hip.linear(x, w, residual=res)[:, cols], want.to(dt), dt, "sampled columns")
    z = (x.float() @ torch.cat([fc[cols], fc[N + cols]]).float().T).to(dt).float()
    want = (F.silu(z[:, :cols.numel()]).to(dt).float() * z[:, cols.numel():]).to(dt)
    check(pkg.hip.linear(x, fc, swiglu=True)[:, cols], want, dt, "sampled columns, SwiGLU")


# ----------------------------------------------------------------------------- attention at 4 x 4096
def test_prefill_attention_config4(pkg):
    """raven_prefill_attention at B=4, S=4096, 55 heads of 96: sampled (sequence, head) pairs against the oracle's sdpa,
    all 4096 query rows of each (the causal case of RMM:484-491)."""
    dt, B, S = torch.bfloat16, 4, 4096
    q = _gpu_randn((B * S, H), 21)
    k = _gpu_randn((1, B, NH, S, HD), 22)
    v = _gpu_randn((1, B, NH, S, HD), 23)
    cache = pkg.hip.make_cache(k, v)
    y = pkg.hip.prefill_attention(q, cache, 0, B, S, 0, NH, HD)
    torch.cuda.synchronize()
    for b, head in ((0, 0), (1, 17), (2, 54), (3, 31), (3, 0)):
        qh = q.view(B, S, NH, HD)[b, :, head].cpu()[None, None]
        want = O.sdpa(qh, k[0, b, head].cpu()[None, None], v[0, b, head].cpu()[None, None])[0, 0]
        check(y.view(B, S, NH, HD)[b, :, head], want, dt, f"sequence {b} head {head}")
    # the chunk kernel and the per-row kernel agree on a sample of rows (two implementations of the same softmax)
    rows = torch.tensor([0, 1, 63, 64, 127, 128, 2047, 2048, 4095])
    for b in (0, 3):
        for r in rows.tolist():
            qr = q.view(B, S, H)[b, r].view(1, NH, 1, HD)
            want = O.sdpa(qr.cpu(), k[0, b, :, :r + 1].cpu()[None], v[0, b, :, :r + 1].cpu()[None]).view(H)
            check(y.view(B, S, H)[b, r], want, dt, f"row {r} of sequence {b}")


def test_prefill_attention_wave_variants_agree(pkg, tuned):
    """head_dim 96 has two workgroup shapes (four waves = 128 query rows, six waves = 192): a row's arithmetic is the same
    in both, so the outputs must be the same bits -- with a chunk length that is no multiple of either, behind cached
    positions, and at the oracle's values on sampled rows."""
    dt, B, S, T0 = torch.bfloat16, 2, 1000, 24
    q = _gpu_randn((B * S, H), 61)
    k = _gpu_randn((1, B, NH, T0 + S, HD), 62)
    v = _gpu_randn((1, B, NH, T0 + S, HD), 63)
    cache = pkg.hip.make_cache(k, v)
    outs = {}
    for waves in (4, 6):
        tuned(prefill_waves=waves)
        outs[waves] = pkg.hip.prefill_attention(q, cache, 0, B, S, T0, NH, HD)
    torch.cuda.synchronize()
    assert torch.equal(outs[4], outs[6])
    for b, r in ((0, 0), (0, 191), (0, 192), (1, 575), (1, 999)):
        qr = q.view(B, S, H)[b, r].view(1, NH, 1, HD)
        want = O.sdpa(qr.cpu(), k[0, b, :, :T0 + r + 1].cpu()[None], v[0, b, :, :T0 + r + 1].cpu()[None]).view(H)
        check(outs[6].view(B, S, H)[b, r], want, dt, f"row {r} of sequence {b}")


# ----------------------------------------------------------------------------- one SandwichBlock at M = 16384
def test_sandwich_block_config4_rows(pkg):
    """raven_sandwich_block on 4 x 4096 rows at the 3.5b dims (tiled products, MFMA chunk attention, fused norms) against
    the oracle's SandwichBlock (RMM:525-536) on sampled rows of one sequence.  The oracle projects K and V for all 4096
    rows of that sequence (attention needs them) and everything else for the sampled rows only."""
    dt, B, S = torch.bfloat16, 4, 4096
    s = O.RavenShape.nebel()
    g = torch.Generator().manual_seed(31)
    prefix = "blk"
    w = {f"{prefix}.norm_{i}.weight": (torch.randn(H, generator=g) * 0.02 + 1).to(dt) for i in (1, 2, 3, 4)}
    w[f"{prefix}.attn.Wqkv.weight"] = (torch.randn(3 * H, H, generator=g) * 0.02).to(dt)
    w[f"{prefix}.attn.qk_bias"] = (torch.randn(2, 1, NH, HD, generator=g) * 0.02).to(dt)
    w[f"{prefix}.attn.proj.weight"] = (torch.randn(H, H, generator=g) * 0.02).to(dt)
    w[f"{prefix}.mlp.fc.weight"] = (torch.randn(2 * INTER, H, generator=g) * 0.02).to(dt)
    w[f"{prefix}.mlp.proj.weight"] = (torch.randn(H, INTER, generator=g) * 0.02).to(dt)
    dev = {k_: v_.cuda() for k_, v_ in w.items()}
    x = _gpu_randn((B * S, H), 32)
    table = O.rope_table(HD, s.block_size, s.rope_base).to(dt)
    freqs = table.float().reshape(s.block_size, HD // 2, 2).contiguous().cuda()
    kd = torch.zeros(1, B, NH, S, HD, dtype=dt, device="cuda")
    vd = torch.zeros_like(kd)
    cache = pkg.hip.make_cache(kd, vd)
    dims = pkg.hip.make_dims(H, NH, INTER, s.norm_eps, dt)
    blk = pkg.hip.make_block_weights(dev[f"{prefix}.norm_1.weight"], dev[f"{prefix}.norm_2.weight"], dev[f"{prefix}.norm_3.weight"],
                                     dev[f"{prefix}.norm_4.weight"], dev[f"{prefix}.attn.Wqkv.weight"], dev[f"{prefix}.attn.qk_bias"],
                                     dev[f"{prefix}.attn.proj.weight"], dev[f"{prefix}.mlp.fc.weight"], dev[f"{prefix}.mlp.proj.weight"])
    ws = pkg.hip.block_workspace(dims, B * S, "cuda")
    out = pkg.hip.sandwich_block(dims, blk, x, torch.empty_like(x), freqs, cache, 0, B, S, 0, ws)
    torch.cuda.synchronize()

    # ---- the oracle, sequence b, fp32-accumulate linears (the same mathematics; the CPU's bf16 GEMM would take minutes)
    b = 2
    rows = torch.tensor([0, 1, 15, 16, 63, 64, 255, 256, 1023, 2048, 3071, 4094, 4095])
    O.set_linear_mode("f32")
    try:
        xb = x.view(B, S, H)[b].cpu()
        n1 = O.rmsnorm(xb, w[f"{prefix}.norm_1.weight"], s.norm_eps)
        wqkv = w[f"{prefix}.attn.Wqkv.weight"]
        kv = O.linear(n1, wqkv[H:])                                     # K and V of every row of the sequence
        k_all, v_all = kv[:, :H].view(1, S, NH, HD), kv[:, H:].view(1, S, NH, HD)
        q_s = O.linear(n1[rows], wqkv[:H]).view(1, -1, NH, HD)          # queries of the sampled rows
        bias = w[f"{prefix}.attn.qk_bias"]
        k_all = (k_all + bias[1:2]).to(dt)
        q_s = (q_s + bias[0:1]).to(dt)
        _, k_rot = O.apply_rope(k_all, k_all, table[:, :S])
        q_rot, _ = O.apply_rope(q_s, q_s, table[:, rows])
        ya = []
        for i, r in enumerate(rows.tolist()):                           # row r attends to positions 0 .. r
            qi = q_rot[:, i:i + 1].transpose(1, 2)
            ya.append(O.sdpa(qi, k_rot[:, :r + 1].transpose(1, 2), v_all[:, :r + 1].transpose(1, 2)).transpose(1, 2).reshape(1, H))
        ya = torch.cat(ya, 0)
        a = O.linear(ya, w[f"{prefix}.attn.proj.weight"])
        x2 = O.rmsnorm(a + xb[rows], w[f"{prefix}.norm_2.weight"], s.norm_eps)
        m = O.gated_mlp(O.rmsnorm(x2, w[f"{prefix}.norm_3.weight"], s.norm_eps), w, prefix)
        want = O.rmsnorm(m + x2, w[f"{prefix}.norm_4.weight"], s.norm_eps)
    finally:
        O.set_linear_mode("native")
    got = out.view(B, S, H)[b][rows.cuda()]
    # the cache rows the block appended: rotated keys and values of every position, one kernel chain deep
    check(kd[0, b].transpose(0, 1), k_rot[0], dt, "appended K of the sequence", ulps=ULPS_COMPOSED)
    check(vd[0, b].transpose(0, 1), v_all[0], dt, "appended V of the sequence")
    err = close(got, want, "block output rows")
    print(f"SandwichBlock at 4 x 4096: sampled rows max-abs {err[0]:.3e} rel-L2 {err[1]:.3e}")
    # a chain of five products and four norms: the composed bar of test_gpu_model.py (per-kernel bars are applied kernel
    # by kernel above and in test_gpu_kernels.py)
    assert err[1] <= 3e-2, f"block output: rel-L2 {err[1]:.3e}"
    scale = max(1.0, want.float().abs().max().item())
    assert err[0] <= 2.5 * 2e-2 * scale, f"block output: max-abs {err[0]:.3e}"
    # rows of other sequences are finite and differ from this one's (no row was skipped or written twice)
    assert torch.isfinite(out.float()).all()
    assert not torch.equal(out.view(B, S, H)[0], out.view(B, S, H)[b])


@pytest.mark.parametrize("nh,hd,B,S,pos0,on_device", [(5, 96, 3, 50, 7, False), (55, 96, 2, 600, 0, True), (22, 128, 4, 512, 3, False),
                                                       (3, 64, 1, 33, 0, False)])
def test_chunk_qkv_epilogue_writes_the_bits_of_the_two_launch_path(pkg, tuned, nh, hd, B, S, pos0, on_device):
    """A chunk's q | k | v product with bias, RoPE and the cache append as its epilogue (fuse_qkv_rope = 1, the default) against
    the stored product followed by raven_qkv_bias_rope_cache_append (RMM:463-481): block output and the K / V rows the block
    appended, bit for bit; likewise with and without padded rows for the activations the tiled GEMM reads (pad_chunk_rows;
    n_embd 480 and 5280 are not multiples of 64).  Shapes: 128 x 128 tiles with rows of three sequences in one tile and heads across tile edges;
    256 x 256 tiles at the 3.5b head layout with the first position on the device; 256 x 256 tiles whose last tile column
    goes to 128 x 128 tiles (2048 rows x 8448 columns: 264 tiles); a single small tile with rows and columns past the end."""
    dt, h, inter = torch.bfloat16, nh * hd, 256
    g = torch.Generator().manual_seed(nh * 1000 + S)
    norms = [(torch.randn(h, generator=g) * 0.02 + 1).to(dt).cuda() for _ in range(4)]
    wqkv = (torch.randn(3 * h, h, generator=g) * 0.02).to(dt).cuda()
    bias = (torch.randn(2, 1, nh, hd, generator=g) * 0.02).to(dt).cuda()
    proj = (torch.randn(h, h, generator=g) * 0.02).to(dt).cuda()
    fc = (torch.randn(2 * inter, h, generator=g) * 0.02).to(dt).cuda()
    mproj = (torch.randn(h, inter, generator=g) * 0.02).to(dt).cuda()
    x = _gpu_randn((B * S, h), 5)
    t_max = pos0 + S + 3
    freqs = O.rope_table(hd, t_max, 50000).to(dt).float().reshape(t_max, hd // 2, 2).contiguous().cuda()
    dims = pkg.hip.make_dims(h, nh, inter, 1e-6, dt)
    blk = pkg.hip.make_block_weights(*norms, wqkv, bias, proj, fc, mproj)
    ws = pkg.hip.block_workspace(dims, B * S, "cuda")
    pos_dev = torch.tensor([pos0], dtype=torch.int32, device="cuda") if on_device else None
    results = []
    for fuse, pad in ((1, 1), (0, 0), (0, 1), (1, 0)):
        tuned(fuse_qkv_rope=fuse, pad_chunk_rows=pad)
        kd = _gpu_randn((2, B, nh, t_max, hd), 6)     # rows outside pos0 .. pos0 + S - 1 must stay as they are
        vd = _gpu_randn((2, B, nh, t_max, hd), 7)
        cache = pkg.hip.make_cache(kd, vd)
        out = pkg.hip.sandwich_block(dims, blk, x, torch.empty_like(x), freqs, cache, 1, B, S, pos0, ws, pos_dev=pos_dev)
        torch.cuda.synchronize()
        results.append((out.clone(), kd, vd))
    (o1, k1, v1), (o0, k0, v0) = results[:2]
    assert torch.equal(k1, k0), "appended K differs between the epilogue and the two-launch path"
    assert torch.equal(v1, v0), "appended V differs"
    assert torch.equal(o1, o0), "block output differs"
    for o, k, v in results[2:]:   # rows of the activations padded to whole cache lines or not, with either q | k | v path
        assert torch.equal(o, o0) and torch.equal(k, k0) and torch.equal(v, v0), "padded activation rows change the result"
    fresh = _gpu_randn((2, B, nh, t_max, hd), 6)
    assert torch.equal(k1[0], fresh[0]) and torch.equal(k1[1, :, :, :pos0], fresh[1, :, :, :pos0]) and torch.equal(k1[1, :, :, pos0 + S:], fresh[1, :, :, pos0 + S:])
    assert not torch.equal(k1[1, :, :, pos0:pos0 + S], fresh[1, :, :, pos0:pos0 + S])


@pytest.mark.parametrize("M,N,K,swiglu", [(300, 5280, 5280, False), (700, 1032, 136, False), (2048, 8448, 2816, False), (1100, 4096, 5280, True),
                                          (40, 64, 72, False)])
def test_packed_weight_copies_change_no_bit(pkg, M, N, K, swiglu):
    """raven_register_packed_weight: a product over 33 and more rows reads the line-aligned copy and writes the bits it
    writes from the matrix itself (both tile sizes, the last tile columns as small tiles, SwiGLU's gate / up rows, a
    K with a partial last step); a matrix that changes must be registered again; after unregistering the matrix is read."""
    hip = pkg.hip
    x = _gpu_randn((M, K), 11)
    w = _gpu_randn((2 * N if swiglu else N, K), 12, std=0.02)
    res = None if swiglu else _gpu_randn((M, N), 13)
    plain = hip.linear(x, w, residual=res, swiglu=swiglu).clone()
    packed = hip.register_packed_weight(w)
    try:
        ld = (K + 63) // 64 * 64
        assert packed.numel() == w.shape[0] * ld * 2
        view = packed.view(torch.bfloat16).view(w.shape[0], ld)
        assert torch.equal(view[:, :K], w) and not view[:, K:].any()
        assert torch.equal(hip.linear(x, w, residual=res, swiglu=swiglu), plain)
        w.mul_(2)                                          # exact in bf16; the copy still holds the old values ...
        assert torch.equal(hip.linear(x, w, residual=res, swiglu=swiglu), plain), "the product did not read the registered copy"
        few = hip.linear(x[:8], w, residual=None if res is None else res[:8], swiglu=swiglu).clone()   # ... which 8 rows never read
        packed2 = hip.register_packed_weight(w)            # ... until the matrix is registered again
        again = hip.linear(x, w, residual=res, swiglu=swiglu).clone()
    finally:
        hip.unregister_packed_weight(w)
    want = hip.linear(x, w, residual=res, swiglu=swiglu)   # the matrix itself
    assert torch.equal(again, want) and not torch.equal(again, plain)
    check(few, want[:8].float(), torch.bfloat16, "8 rows against the first rows of the large product", ulps=ULPS_SWIGLU if swiglu else ULPS_RESIDUAL)
    del packed, packed2


def test_bench_prefill_iteration_runs_through_the_c_abi(pkg):
    """One recurrence over 4 x 512 rows through raven_core_iteration (adapter with two K segments, four blocks, chunk
    attention over a cache that already holds 512 positions): determinism, and the call equals adapter + four
    raven_sandwich_block calls bit for bit (one composition of the block behind the C ABI)."""
    dt, B, S, T = torch.bfloat16, 4, 512, 512
    s = O.RavenShape.nebel()
    w = O.make_weights(s, seed=0, dtype=dt, only_core=True)
    dev = {k_: v_.cuda() for k_, v_ in w.items()}
    from test_gpu_model import _block_weights
    blocks = (pkg.hip.BlockWeights * 4)(*[_block_weights(pkg, dev, f"transformer.core_block.{j}") for j in range(4)])
    dims = pkg.hip.make_dims(H, NH, INTER, s.norm_eps, dt)
    table = O.rope_table(HD, s.block_size, s.rope_base).to(dt)
    freqs = table.float().reshape(s.block_size, HD // 2, 2).contiguous().cuda()
    state, embeds = _gpu_randn((B * S, H), 41, 0.632), _gpu_randn((B * S, H), 42)
    k0, v0 = _gpu_randn((4, B, NH, T + S, HD), 43), _gpu_randn((4, B, NH, T + S, HD), 44)
    ws = pkg.hip.block_workspace(dims, B * S, "cuda")
    outs = []
    for _ in range(2):
        kd, vd = k0.clone(), v0.clone()
        out = torch.empty_like(state)
        pkg.hip.core_iteration(dims, dev["transformer.adapter.weight"], blocks, state, embeds, out, freqs, pkg.hip.make_cache(kd, vd), 0, B, S,
                               T, ws)
        outs.append((out, kd, vd))
    assert all(torch.equal(a, b) for a, b in zip(outs[0], outs[1]))
    kd, vd = k0.clone(), v0.clone()
    cache = pkg.hip.make_cache(kd, vd)
    cur = pkg.hip.linear(state, dev["transformer.adapter.weight"], x1=embeds)
    for j in range(4):
        nxt = torch.empty_like(cur)
        pkg.hip.sandwich_block(dims, blocks[j], cur, nxt, freqs, cache, j, B, S, T, ws)
        cur = nxt
    assert torch.equal(cur, outs[0][0]) and torch.equal(kd, outs[0][1]) and torch.equal(vd, outs[0][2])
    assert torch.isfinite(cur.float()).all()
