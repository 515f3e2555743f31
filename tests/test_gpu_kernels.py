"""GPU parity tests, kernel by kernel, through the C ABI (pkg.hip wrappers are thin ctypes calls)
against the CPU oracle on identical seeded inputs.

Tolerances: bf16 results must satisfy max-abs <= 2e-2 and rel-L2 <= 1e-2 against the oracle
(the bar the build's target states for per-kernel outputs), element by element; an element whose
reference value is 4 or larger, where one step of bf16 is already 0.031, may instead be one step off.
fp32 results 1e-4 / 1e-5; integer outputs (argmax ids, cache positions) bit-exact.  The largest
max-abs and rel-L2 every test saw are printed at the end of the run."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import raven_oracle as O

pytestmark = pytest.mark.gpu

BF16_MAXABS, BF16_RELL2 = 2e-2, 1e-2
F32_MAXABS, F32_RELL2 = 1e-4, 1e-5


def close(got: torch.Tensor, want: torch.Tensor, what: str = ""):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    max_abs = (got - want).abs().max().item()
    rel = ((got - want).norm() / want.norm().clamp_min(1e-30)).item()
    return max_abs, rel


PARITY_LOG = {}  # test id -> [largest max-abs, largest rel-L2, checks]; printed by conftest's terminal summary


def bf16_spacing(t: torch.Tensor) -> torch.Tensor:
    """Distance between neighbouring bf16 values at each element's magnitude (8 significant bits)."""
    a = t.detach().float().abs().clamp_min(2.0 ** -126)
    return torch.exp2(torch.floor(torch.log2(a)) - 7)


ULPS_SWIGLU = 3    # silu(gate) * up: two rounded factors, each of which may land one step off, and the product's own rounding
# round(round(product) + residual): sums of bf16 products land on exact ties of the bf16 grid often; when the product is a
# tie the two implementations' fp32 sums may break it differently (one step), and the sum with the residual is then a tie
# again whose two break directions lie one more step apart (seen: -6.140625 -> -6.125 / -6.15625, + 1.671875 -> -4.4375 / -4.5)
ULPS_RESIDUAL = 2
# results behind several kernels in a row (a block, a small model's forward): an element's error no longer scales with the
# element but with the sums it came from, so the step is taken at the largest magnitude of the element's row; four such
# steps (largest seen: three, in the small bf16 models' latents behind 6 to 14 blocks)
ULPS_COMPOSED = "4 steps at the row's largest magnitude"


def check(got, want, dtype, what="", ulps=1, mag=None):
    """bf16: every element within 2e-2 of the reference element or, where the reference element is so large that bf16
    cannot resolve 2e-2 (|ref| >= 4: one step of the format is 0.031), within `ulps` steps of the format there; and
    rel-L2 <= 1e-2.  `mag`: an intermediate that was rounded to bf16 on the way (the product in front of a residual add,
    RMM:534-535); the step is then taken at the larger of the two magnitudes, since a one-step flip of the product
    survives a cancelling add.  fp32: max-abs 1e-4 (times the largest reference magnitude when that exceeds 1), rel-L2 1e-5."""
    max_abs, rel = close(got, want, what)
    import os
    rec = PARITY_LOG.setdefault(os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0], [0.0, 0.0, 0])
    rec[0], rec[1], rec[2] = max(rec[0], max_abs), max(rec[1], rel), rec[2] + 1
    if dtype == torch.bfloat16:
        g, w = got.detach().float().cpu(), want.detach().float().cpu()
        if ulps == ULPS_COMPOSED:
            ulps, at = 4, w.abs().amax(dim=-1, keepdim=True).expand_as(w)
        else:
            at = w if mag is None else torch.maximum(w.abs(), mag.detach().float().cpu().abs())
        bar = (ulps * bf16_spacing(at)).clamp_min(BF16_MAXABS)
        over = (g - w).abs() > bar
        worst = ((g - w).abs() / bar).max().item() if g.numel() else 0.0
        assert not over.any() and rel <= BF16_RELL2, \
            f"{what}: max-abs {max_abs:.3e}, {int(over.sum())} elements beyond max(2e-2, {ulps} bf16 ulp) (worst {worst:.2f} x the bar), rel-L2 {rel:.3e}"
    else:
        scale = max(1.0, want.detach().float().abs().max().item())
        assert max_abs <= F32_MAXABS * scale and rel <= F32_RELL2, f"{what}: max-abs {max_abs:.3e} (scale {scale:.2f}), rel-L2 {rel:.3e}"


def rnd(shape, dtype, seed, std=1.0, mean=0.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std + mean).to(dtype)


# ----------------------------------------------------------------------------- RMSNorm (config 2)
@pytest.mark.parametrize("rows", [1, 32, 4096])
def test_rmsnorm_residual_bf16_5280(pkg, rows):
    dt, n = torch.bfloat16, 5280
    x, res = rnd((rows, n), dt, 1), rnd((rows, n), dt, 2)
    w = rnd((n,), dt, 3, 0.02, 1.0)
    y, s, _ = pkg.hip.rmsnorm_residual(x.cuda(), w.cuda(), 1e-6, residual=res.cuda(), want_sum=True)
    want_sum = x + res
    assert torch.equal(s.cpu(), want_sum), "residual sum must be bit-exact (one bf16 add)"
    check(y, O.rmsnorm(want_sum, w, 1e-6), dt, f"rmsnorm+residual rows={rows}")
    # against an fp32-accumulate torch statement of the same op
    ref32 = (F.rms_norm(want_sum.float(), (n,), eps=1e-6).to(dt).float() * w.float())
    check(y, ref32, dt, "rmsnorm vs F.rms_norm")
    # without a residual, and the fraction of bit-identical outputs should be overwhelming
    y2, _, _ = pkg.hip.rmsnorm_residual(x.cuda(), w.cuda(), 1e-6)
    want = O.rmsnorm(x, w, 1e-6)
    check(y2, want, dt, "rmsnorm")
    assert (y2.cpu() == want).float().mean().item() > 0.999


def test_rmsnorm_double_and_fp32_and_ragged_dims(pkg):
    for dt, n, rows in ((torch.float32, 256, 7), (torch.bfloat16, 5280, 3), (torch.bfloat16, 8, 2), (torch.float32, 4, 1),
                        (torch.bfloat16, 8192, 2)):
        x = rnd((rows, n), dt, 5)
        w1, w2 = rnd((n,), dt, 6, 0.02, 1.0), rnd((n,), dt, 7, 0.02, 1.0)
        y, _, y2 = pkg.hip.rmsnorm_residual(x.cuda(), w1.cuda(), 1e-6, weight2=w2.cuda())
        want1 = O.rmsnorm(x, w1, 1e-6)
        check(y, want1, dt, f"norm {dt} {n}")
        check(y2, O.rmsnorm(want1, w2, 1e-6), dt, f"double norm {dt} {n}")
    # closed form: constant rows
    xc = torch.full((2, 5280), 3.0, dtype=torch.bfloat16)
    y, _, _ = pkg.hip.rmsnorm_residual(xc.cuda(), torch.ones(5280, dtype=torch.bfloat16).cuda(), 1e-6)
    assert torch.equal(y.cpu(), torch.ones(2, 5280, dtype=torch.bfloat16))
    # empty input and bad sizes
    e, _, _ = pkg.hip.rmsnorm_residual(torch.empty(0, 256, device="cuda"), torch.ones(256, device="cuda"), 1e-6)
    assert e.shape == (0, 256)
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.rmsnorm_residual(torch.zeros(1, 6, device="cuda"), torch.ones(6, device="cuda"), 1e-6)


# ----------------------------------------------------------------------------- skinny GEMMs
def lin(x, w):
    return F.linear(x.float(), w.float())


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 16, 17, 32, 33, 70])
def test_gemm_bf16_all_row_counts(pkg, M):
    dt, N, K = torch.bfloat16, 528, 1056
    x, w = rnd((M, K), dt, 10 + M), rnd((N, K), dt, 20, 0.05)
    res = rnd((M, N), dt, 30)
    y = pkg.hip.gemm(x.cuda(), w.cuda())
    check(y, lin(x, w).to(dt), dt, f"gemm M={M}")
    yr = pkg.hip.gemm(x.cuda(), w.cuda(), residual=res.cuda())
    check(yr, (lin(x, w).to(dt) + res), dt, f"gemm+residual M={M}", mag=lin(x, w), ulps=ULPS_RESIDUAL)
    yf = pkg.hip.gemm(x.cuda(), w.cuda(), out_f32=True)
    assert yf.dtype == torch.float32
    assert torch.equal(yf.cpu(), y.float().cpu()), "float store must be the upcast of the rounded result"


@pytest.mark.parametrize("M", [1, 2, 3, 4, 8, 32])
@pytest.mark.parametrize("N,K", [(5280, 5280), (15840, 5280), (5280, 17920)])
def test_gemm_bf16_nebel_shapes(pkg, M, N, K):
    dt = torch.bfloat16
    x, w = rnd((M, K), dt, 40 + M), rnd((N, K), dt, 41, 0.02)
    y = pkg.hip.gemm(x.cuda(), w.cuda())
    check(y, lin(x, w).to(dt), dt, f"gemm {M}x{N}x{K}")


@pytest.mark.parametrize("M", [1, 8, 32])
def test_lm_head_product_at_decode_row_counts(pkg, M):
    """The LM head of a decode step: [M, 5280] x [65536, 5280]^T with the float store (logits stay fp32, RMM:712-714),
    at 1, 8 and 32 rows -- the widest product of a token (692 MB of weights, 32768 workgroups of the one-row kernel).
    Against fp32 F.linear on the first and last 1024 vocabulary rows and 2048 rows in between."""
    dt, N, K = torch.bfloat16, 65536, 5280
    x = rnd((M, K), dt, 60 + M)
    wd = torch.empty(N, K, dtype=dt, device="cuda").normal_(0.0, 0.02, generator=torch.Generator(device="cuda").manual_seed(61))
    y = pkg.hip.gemm(x.cuda(), wd, out_f32=True)
    assert y.dtype == torch.float32 and y.shape == (M, N)
    cols = torch.cat([torch.arange(1024), torch.randperm(N - 2048, generator=torch.Generator().manual_seed(62))[:2048] + 1024,
                      torch.arange(N - 1024, N)])
    want = lin(x, wd[cols.cuda()].cpu()).to(dt)
    check(y[:, cols.cuda()], want, dt, f"LM head M={M}")
    assert torch.equal(y, y.to(dt).float()), "the float store holds the bf16-rounded product"
    # every vocabulary row was written: the product against the device's own fp32 matmul over all 65536 columns
    full = (x.cuda().float() @ wd.float().t()).to(dt)
    check(y, full, dt, f"LM head M={M}, all columns")


def test_embedding_at_the_full_vocabulary(pkg):
    """raven_embed over the 65536 x 5280 table: first, last and random rows, scaled by sqrt(5280) in the table's dtype
    (one rounding, RMM:672-675)."""
    dt, V, h = torch.bfloat16, 65536, 5280
    wd = torch.empty(V, h, dtype=dt, device="cuda").normal_(0.0, 0.02, generator=torch.Generator(device="cuda").manual_seed(63))
    ids = torch.cat([torch.tensor([0, V - 1, 1, V - 2, 32768]), torch.randint(0, V, (59,), generator=torch.Generator().manual_seed(64))])
    scale = math.sqrt(h)
    got = pkg.hip.embed(wd, ids.cuda(), scale)
    want = (wd[ids.cuda()].cpu() * scale)   # a bf16 tensor times a Python float: computed in fp32, rounded once
    assert got.shape == (64, h) and torch.equal(got.cpu(), want)
    wf = wd[:4096].float()
    gf = pkg.hip.embed(wf, torch.tensor([0, 4095, 17]).cuda(), scale)
    assert torch.equal(gf.cpu(), (wf[[0, 4095, 17]].cpu() * scale))


@pytest.mark.parametrize("M", [1, 3, 8, 9, 40])
def test_gemm_fp32_tiny_shapes(pkg, M):
    dt = torch.float32
    for N, K in ((768, 256), (256, 256), (256, 704), (1024, 256), (6, 4)):
        x, w = rnd((M, K), dt, 50), rnd((N, K), dt, 51, 0.1)
        check(pkg.hip.gemm(x.cuda(), w.cuda()), lin(x, w), dt, f"fp32 gemm {M}x{N}x{K}")


@pytest.mark.parametrize("dt,M,h", [(torch.bfloat16, 1, 5280), (torch.bfloat16, 32, 5280), (torch.bfloat16, 6, 64),
                                    (torch.float32, 1, 256), (torch.float32, 12, 256)])
def test_adapter_concat(pkg, dt, M, h):
    x0, x1 = rnd((M, h), dt, 60), rnd((M, h), dt, 61)
    w = rnd((h, 2 * h), dt, 62, 0.02)
    y = pkg.hip.adapter_gemm_concat(x0.cuda(), x1.cuda(), w.cuda())
    want = lin(torch.cat([x0, x1], -1), w).to(dt)
    check(y, want, dt, "adapter (state, embeds)")
    swapped = lin(torch.cat([x1, x0], -1), w).to(dt)
    assert close(y, swapped)[1] > 0.1, "operand order must matter"


@pytest.mark.parametrize("dt,M,I,K", [(torch.bfloat16, 1, 17920, 5280), (torch.bfloat16, 32, 17920, 5280),
                                      (torch.bfloat16, 8, 17920, 5280), (torch.bfloat16, 3, 176, 64),
                                      (torch.float32, 1, 704, 256), (torch.float32, 20, 704, 256)])
def test_gemm_swiglu(pkg, dt, M, I, K):
    x, fc = rnd((M, K), dt, 70), rnd((2 * I, K), dt, 71, 0.03)
    y = pkg.hip.gemm_swiglu(x.cuda(), fc.cuda())
    z = lin(x, fc).to(dt)
    gate, up = z[:, :I], z[:, I:]
    want = F.silu(gate) * up
    check(y, want, dt, "swiglu", ulps=ULPS_SWIGLU)
    wrong = F.silu(up) * gate
    assert close(y, wrong)[1] > 0.1, "the gate must be the first half"


@pytest.mark.parametrize("M", [2, 3, 4, 5, 8, 16, 17, 32, 33, 34, 40])
@pytest.mark.parametrize("ks", [0, 3])
def test_linear_with_workspace_nebel_shapes(pkg, tuned, M, ks):
    """raven_linear at the 3.5b shapes, every epilogue: with the library's own choice between its two MFMA
    kernels (ks = 0) and with the split-K, shared-X kernel forced to three K slices for every matrix."""
    dt, h, I = torch.bfloat16, 5280, 17920
    tuned(linear_ks=ks)
    ws = pkg.hip.linear_workspace(M, 2 * I, "cuda")
    x, xi, x1 = rnd((M, h), dt, 160 + M), rnd((M, I), dt, 161), rnd((M, h), dt, 162)
    res = rnd((M, h), dt, 163)
    wqkv, proj, fc, mlp, ada = (rnd(sh, dt, 164 + i, 0.02) for i, sh in enumerate(((3 * h, h), (h, h), (2 * I, h), (h, I), (h, 2 * h))))
    dev = lambda t: t.cuda()
    check(pkg.hip.linear(dev(x), dev(wqkv), workspace=ws), lin(x, wqkv).to(dt), dt, "qkv")
    check(pkg.hip.linear(dev(x), dev(proj), residual=dev(res), workspace=ws), lin(x, proj).to(dt) + res, dt, "proj + residual", mag=lin(x, proj), ulps=ULPS_RESIDUAL)
    z = lin(x, fc).to(dt)
    check(pkg.hip.linear(dev(x), dev(fc), swiglu=True, workspace=ws), F.silu(z[:, :I]) * z[:, I:], dt, "fc + swiglu", ulps=ULPS_SWIGLU)
    check(pkg.hip.linear(dev(xi), dev(mlp), residual=dev(res), workspace=ws), lin(xi, mlp).to(dt) + res, dt, "mlp.proj + residual", mag=lin(xi, mlp), ulps=ULPS_RESIDUAL)
    check(pkg.hip.linear(dev(x), dev(ada), x1=dev(x1), workspace=ws), lin(torch.cat([x, x1], -1), ada).to(dt), dt, "adapter")
    yf = pkg.hip.linear(dev(x), dev(proj), out_f32=True, workspace=ws)
    assert yf.dtype == torch.float32 and torch.equal(yf, pkg.hip.linear(dev(x), dev(proj), workspace=ws).float())
    # the same call twice gives the same bits (partials are added in a fixed order), and no workspace gives the same values
    a, b = pkg.hip.linear(dev(xi), dev(mlp), workspace=ws), pkg.hip.linear(dev(xi), dev(mlp), workspace=ws)
    assert torch.equal(a, b)
    check(pkg.hip.linear(dev(xi), dev(mlp)), lin(xi, mlp).to(dt), dt, "no workspace")


def test_linear_small_and_odd_shapes(pkg, tuned):
    dt = torch.bfloat16
    tuned(linear_ks=2)  # the split-K kernel for everything it accepts
    for M, N, K in ((9, 48, 160), (32, 16, 128), (12, 528, 1056), (7, 32, 96), (6, 20, 64)):
        x, w = rnd((M, K), dt, 170), rnd((N, K), dt, 171, 0.05)
        ws = pkg.hip.linear_workspace(M, N, "cuda")
        check(pkg.hip.linear(x.cuda(), w.cuda(), workspace=ws), lin(x, w).to(dt), dt, f"linear {M}x{N}x{K}")
    x, w = rnd((3, 256), torch.float32, 172), rnd((64, 256), torch.float32, 173, 0.1)
    check(pkg.hip.linear(x.cuda(), w.cuda(), workspace=pkg.hip.linear_workspace(3, 64, "cuda")), lin(x, w), torch.float32, "fp32 falls through")


@pytest.mark.parametrize("M", [6, 20])
@pytest.mark.parametrize("four", [1, 2])
def test_mfma_gemm_row_alignment_cases(pkg, tuned, M, four):
    """Row pitches that are odd multiples of 64 bytes (tiles of one row parity, macro-steps shifted to the line
    boundary), with and without whole tile pairs, a second operand that starts mid-line, and a weight matrix
    whose base address is not line-aligned; both MFMA kernels (with and without a workspace)."""
    dt = torch.bfloat16
    ws = pkg.hip.linear_workspace(M, 4096, "cuda")
    # four = 2: the four-tile, 64-wide-step variant wherever there is no workspace; with a workspace: the split-K kernel
    tuned(gemm_four_tiles=four, linear_ks=2)
    for N, K in ((32, 96), (64, 288), (64, 2336), (96, 416), (48, 416), (160, 1184), (64, 256)):
        x, w = rnd((M, K), dt, 180 + N), rnd((N, K), dt, 181 + K, 0.05)
        want = lin(x, w).to(dt)
        for wsp in (None, ws):
            check(pkg.hip.linear(x.cuda(), w.cuda(), workspace=wsp), want, dt, f"plain {M}x{N}x{K} ws={wsp is not None}")
        # the same matrix 16 bytes into an allocation
        flat = torch.zeros(N * K + 8, dtype=dt, device="cuda")
        flat[8:] = w.cuda().reshape(-1)
        for wsp in (None, ws):
            check(pkg.hip.linear(x.cuda(), flat[8:].view(N, K), workspace=wsp), want, dt, f"offset base {M}x{N}x{K}")
    for I, K in ((64, 160), (96, 416), (48, 288)):
        x, fc = rnd((M, K), dt, 190), rnd((2 * I, K), dt, 191 + I, 0.05)
        z = lin(x, fc).to(dt)
        for wsp in (None, ws):
            check(pkg.hip.linear(x.cuda(), fc.cuda(), swiglu=True, workspace=wsp), F.silu(z[:, :I]) * z[:, I:], dt, f"swiglu {M}x{I}x{K}", ulps=ULPS_SWIGLU)
    for N, K0, K1 in ((64, 160, 160), (32, 288, 160), (64, 416, 416)):
        x0, x1, w = rnd((M, K0), dt, 195), rnd((M, K1), dt, 196), rnd((N, K0 + K1), dt, 197 + N, 0.05)
        for wsp in (None, ws):
            check(pkg.hip.linear(x0.cuda(), w.cuda(), x1=x1.cuda(), workspace=wsp), lin(torch.cat([x0, x1], -1), w).to(dt), dt,
                  f"two operands {M}x{N}x({K0}+{K1})")


@pytest.mark.parametrize("M", [8, 32])
def test_mfma_four_tile_variant_nebel_shapes(pkg, tuned, M):
    dt, h, I = torch.bfloat16, 5280, 17920
    tuned(gemm_four_tiles=2)
    x, xi, res = rnd((M, h), dt, 230 + M), rnd((M, I), dt, 231), rnd((M, h), dt, 232)
    wqkv, fc, mlp = rnd((3 * h, h), dt, 233, 0.02), rnd((2 * I, h), dt, 234, 0.02), rnd((h, I), dt, 235, 0.02)
    check(pkg.hip.gemm(x.cuda(), wqkv.cuda()), lin(x, wqkv).to(dt), dt, "qkv")
    z = lin(x, fc).to(dt)
    check(pkg.hip.gemm_swiglu(x.cuda(), fc.cuda()), F.silu(z[:, :I]) * z[:, I:], dt, "fc + swiglu", ulps=ULPS_SWIGLU)
    check(pkg.hip.gemm(xi.cuda(), mlp.cuda(), residual=res.cuda()), lin(xi, mlp).to(dt) + res, dt, "mlp.proj + residual", mag=lin(xi, mlp), ulps=ULPS_RESIDUAL)
    yf = pkg.hip.gemm(x.cuda(), wqkv.cuda(), out_f32=True)
    assert yf.dtype == torch.float32 and torch.equal(yf, pkg.hip.gemm(x.cuda(), wqkv.cuda()).float())


@pytest.mark.parametrize("dt,h,I", [(torch.bfloat16, 5280, 17920), (torch.float32, 256, 704), (torch.bfloat16, 64, 176)])
def test_gemv_fused_one_row(pkg, dt, h, I):
    """The one-row kernel with its norm prologues and epilogues, against the oracle's separate ops."""
    x = rnd((h,), dt, 120)
    wa, wb = rnd((h,), dt, 121, 0.02, 1.0), rnd((h,), dt, 122, 0.02, 1.0)
    res = rnd((h,), dt, 123)
    wqkv, fc, mlp = rnd((3 * h, h), dt, 124, 0.02), rnd((2 * I, h), dt, 125, 0.03), rnd((h, I), dt, 126, 0.02)
    ada, x1 = rnd((h, 2 * h), dt, 127, 0.02), rnd((h,), dt, 128)
    xa_want = O.rmsnorm(x[None], wa, 1e-6)
    xb_want = O.rmsnorm(xa_want, wb, 1e-6)
    dev = lambda t: t.cuda()
    # norm_4 -> norm_1 -> Wqkv, with the first norm written out
    y, xa = pkg.hip.gemv_fused(dev(x), dev(wqkv), norm_a=dev(wa), norm_b=dev(wb), want_xa=True)
    check(xa[None], xa_want, dt, "norm_a output")
    check(y[None], lin(xb_want, wqkv).to(dt), dt, "double norm + qkv")
    # single norm, no store
    y, _ = pkg.hip.gemv_fused(dev(x), dev(wqkv), norm_a=dev(wa))
    check(y[None], lin(xa_want, wqkv).to(dt), dt, "norm + qkv")
    # norm_2 -> norm_3 -> fc with SwiGLU
    y, xa = pkg.hip.gemv_fused(dev(x), dev(fc), norm_a=dev(wa), norm_b=dev(wb), want_xa=True, swiglu=True)
    z = lin(xb_want, fc).to(dt)
    check(y[None], F.silu(z[:, :I]) * z[:, I:], dt, "double norm + fc + swiglu", ulps=ULPS_SWIGLU)
    # long K with residual (mlp.proj) and the adapter's two operands
    g = rnd((I,), dt, 129)
    y, _ = pkg.hip.gemv_fused(dev(g), dev(mlp), residual=dev(res))
    check(y[None], lin(g[None], mlp).to(dt) + res, dt, "mlp.proj + residual", mag=lin(g[None], mlp), ulps=ULPS_RESIDUAL)
    y, _ = pkg.hip.gemv_fused(dev(x), dev(ada), x1=dev(x1))
    check(y[None], lin(torch.cat([x, x1])[None], ada).to(dt), dt, "adapter")
    y, _ = pkg.hip.gemv_fused(dev(x), dev(ada), x1=dev(x1), norm_a=dev(wa))
    check(y[None], lin(torch.cat([xa_want[0], x1])[None], ada).to(dt), dt, "norm on the first operand only")
    yf, _ = pkg.hip.gemv_fused(dev(x), dev(wqkv), out_f32=True)
    y, _ = pkg.hip.gemv_fused(dev(x), dev(wqkv))
    assert yf.dtype == torch.float32 and torch.equal(yf, y.float())
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.gemv_fused(dev(x), dev(wqkv), norm_b=dev(wb))  # norm_b without norm_a


# ----------------------------------------------------------------------------- RoPE + cache append
def make_cache(pkg, n_slots, B, nh, t_max, hd, dt, fill_seed=None):
    if fill_seed is None:
        k = torch.zeros(n_slots, B, nh, t_max, hd, dtype=dt)
        v = torch.zeros_like(k)
    else:
        k, v = rnd((n_slots, B, nh, t_max, hd), dt, fill_seed), rnd((n_slots, B, nh, t_max, hd), dt, fill_seed + 1)
    kd, vd = k.cuda(), v.cuda()
    return k, v, kd, vd, pkg.hip.make_cache(kd, vd)


@pytest.mark.parametrize("dt,nh,hd,B,S,pos0", [(torch.bfloat16, 55, 96, 1, 1, 1023), (torch.bfloat16, 55, 96, 4, 3, 7),
                                               (torch.float32, 4, 64, 2, 5, 0), (torch.bfloat16, 2, 128, 1, 2, 3)])
def test_qkv_bias_rope_cache_append(pkg, dt, nh, hd, B, S, pos0):
    h, t_max, slot = nh * hd, 1024, 2
    qkv = rnd((B * S, 3 * h), dt, 80)
    bias = rnd((2, 1, nh, hd), dt, 81, 0.5)
    table = O.rope_table(hd, t_max, 50000.0).to(dt)  # the table as a dtype-cast module holds it
    freqs = table.float().reshape(t_max, hd // 2, 2).contiguous()
    k0, v0, kd, vd, cache = make_cache(pkg, 4, B, nh, t_max, hd, dt, fill_seed=82)
    q = pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs.cuda(), cache, slot, B, S, pos0, nh, hd)
    # oracle: the same lines of the attention function
    qq, kk, vv = (t.view(B, S, nh, hd) for t in qkv.view(B, S, 3 * h).split([h, h, h], dim=2))
    qq, kk = (qq + bias[0:1]).to(dt), (kk + bias[1:2]).to(dt)
    rq, rk = O.apply_rope(qq, kk, table[:, pos0:pos0 + S])
    check(q.view(B, S, nh, hd), rq, dt, "rotated q")
    got_k = kd[slot, :, :, pos0:pos0 + S].cpu()
    got_v = vd[slot, :, :, pos0:pos0 + S].cpu()
    check(got_k, rk.transpose(1, 2), dt, "cached k")
    assert torch.equal(got_v, vv.transpose(1, 2)), "v is copied unchanged"
    if dt == torch.bfloat16:  # same rounding points: nearly every bf16 value is bit-identical
        assert bool((q.view(B, S, nh, hd).cpu() == rq).float().mean() > 0.995)
    # nothing outside the written window changed: indexing is bit-exact
    kd2, vd2 = kd.cpu(), vd.cpu()
    kd2[slot, :, :, pos0:pos0 + S] = k0[slot, :, :, pos0:pos0 + S]
    vd2[slot, :, :, pos0:pos0 + S] = v0[slot, :, :, pos0:pos0 + S]
    assert torch.equal(kd2, k0) and torch.equal(vd2, v0)
    # negative slot indexes from the end; device-side position overrides the by-value one
    pos_dev = torch.tensor([pos0], dtype=torch.int32, device="cuda")
    pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs.cuda(), cache, -1, B, S, t_max - S, nh, hd, pos_dev=pos_dev)
    assert torch.equal(kd[3, :, :, pos0:pos0 + S].cpu(), got_k)
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs.cuda(), cache, 4, B, S, pos0, nh, hd)
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs.cuda(), cache, 0, B, S, t_max, nh, hd)


# ----------------------------------------------------------------------------- decode attention
@pytest.mark.parametrize("dt,nh,hd,B,S,pos0", [
    (torch.bfloat16, 55, 96, 1, 1, 1023),   # config 3, bs=1: 1024 cached positions
    (torch.bfloat16, 55, 96, 32, 1, 1023),  # config 3, bs=32 (no split)
    (torch.bfloat16, 55, 96, 1, 1, 0),      # a single key: output equals v
    (torch.bfloat16, 55, 96, 2, 1, 70),
    (torch.bfloat16, 55, 96, 1, 6, 200),    # chunk of 6 queries, lower-right causal
    (torch.float32, 4, 64, 1, 1, 11),
    (torch.float32, 4, 64, 2, 8, 0),        # prefill from an empty cache: plain causal
    (torch.bfloat16, 3, 128, 1, 1, 300),
])
def test_decode_attention(pkg, dt, nh, hd, B, S, pos0):
    t_max = 1024
    k, v, kd, vd, cache = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=90)
    q = rnd((B * S, nh * hd), dt, 92)
    ws = pkg.hip.attention_workspace(B * S, nh, hd, "cuda")
    y = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd, workspace=ws)
    T = pos0 + S
    qq = q.view(B, S, nh, hd).transpose(1, 2)
    want = O.sdpa(qq, k[1, :, :, :T], v[1, :, :, :T]).transpose(1, 2).reshape(B * S, nh * hd)
    check(y, want, dt, f"attention B={B} S={S} T={T}")
    lib = F.scaled_dot_product_attention(qq.float(), k[1, :, :, :T].float(), v[1, :, :, :T].float(),
                                         attn_mask=None if S == 1 else torch.ones(S, T, dtype=torch.bool).tril(T - S))
    check(y, lib.transpose(1, 2).reshape(B * S, nh * hd), dt, "attention vs torch SDPA")
    if T == 1:
        check(y.view(B, nh, hd), v[1, :, :, 0], dt, "T=1 returns v")
    # the device-side position overrides the by-value one
    pos_dev = torch.tensor([pos0], dtype=torch.int32, device="cuda")
    y2 = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, t_max - S, nh, hd, pos_dev=pos_dev, workspace=ws)
    check(y2, want, dt, "attention, device-side position (the split count follows the by-value hint)")
    # without a workspace nothing is split; same values up to the order of the merge
    y3 = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd)
    check(y3, want, dt, "attention without workspace")


@pytest.mark.parametrize("B,S,pos0,t_max,nosplit_len", [(3, 1, 1900, 2048, None), (2, 1, 70, 1024, 0), (1, 6, 200, 1024, 0),
                                                        (4, 1, 1023, 1024, 0), (2, 1, 1023, 1024, None)])
def test_decode_attention_of_several_rows_split_and_unsplit(pkg, tuned, B, S, pos0, t_max, nosplit_len):
    """Two rows and more over the contiguous cache: split over positions by the library's rule (a long cache) or because
    the length rule is switched off, and one workgroup per (head, row) otherwise; each against the oracle."""
    dt, nh, hd = torch.bfloat16, 55, 96
    k, v, kd, vd, cache = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=95)
    q = rnd((B * S, nh * hd), dt, 96)
    T = pos0 + S
    want = O.sdpa(q.view(B, S, nh, hd).transpose(1, 2), k[1, :, :, :T], v[1, :, :, :T]).transpose(1, 2).reshape(B * S, nh * hd)
    ws = pkg.hip.attention_workspace(B * S, nh, hd, "cuda")
    if nosplit_len is not None:
        tuned(attn_nosplit_len=nosplit_len)
    y = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd, workspace=ws)
    check(y, want, dt, f"attention B={B} S={S} T={T}, length rule {nosplit_len}")
    tuned(attn_nosplit_len=1 << 20)   # never split two rows and more
    y1 = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd, workspace=ws)
    check(y1, want, dt, f"attention B={B} S={S} T={T}, one workgroup per (head, row)")


@pytest.mark.parametrize("dt,nh,hd,B,pos0", [(torch.bfloat16, 55, 96, 1, 1023), (torch.bfloat16, 55, 96, 32, 600),
                                             (torch.bfloat16, 55, 96, 1, 0), (torch.float32, 4, 64, 3, 17),
                                             (torch.bfloat16, 2, 128, 2, 130)])
def test_qkv_attention_decode_fused(pkg, dt, nh, hd, B, pos0):
    """The one-launch decode step equals append-then-attend, and both equal the oracle."""
    h, t_max = nh * hd, 1024
    qkv = rnd((B, 3 * h), dt, 110)
    bias = rnd((2, 1, nh, hd), dt, 111, 0.5)
    table = O.rope_table(hd, t_max, 50000.0).to(dt)
    freqs = table.float().reshape(t_max, hd // 2, 2).contiguous().cuda()
    k, v, kd, vd, cache = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=112)
    k2, v2, kd2, vd2, cache2 = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=112)
    ws = pkg.hip.attention_workspace(B, nh, hd, "cuda")
    y = pkg.hip.qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, cache, 1, B, pos0, nh, hd, workspace=ws)
    q = pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs, cache2, 1, B, 1, pos0, nh, hd)
    y_two = pkg.hip.decode_attention(q, cache2, 1, B, 1, pos0, nh, hd, workspace=ws)
    assert torch.equal(kd, kd2) and torch.equal(vd, vd2), "fused and two-step paths must write the same cache bytes"
    check(y, y_two, dt, "fused vs two-step")
    qq, kk, vv = (t.view(B, 1, nh, hd) for t in qkv.view(B, 1, 3 * h).split([h, h, h], dim=2))
    qq, kk = (qq + bias[0:1]).to(dt), (kk + bias[1:2]).to(dt)
    rq, rk = O.apply_rope(qq, kk, table[:, pos0:pos0 + 1])
    K = torch.cat([k[1, :, :, :pos0], rk.transpose(1, 2)], dim=2)
    V = torch.cat([v[1, :, :, :pos0], vv.transpose(1, 2)], dim=2)
    want = O.sdpa(rq.transpose(1, 2), K, V).transpose(1, 2).reshape(B, h)
    check(y, want, dt, "fused decode attention vs oracle")
    pos_dev = torch.tensor([pos0], dtype=torch.int32, device="cuda")
    y3 = pkg.hip.qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, cache, 1, B, t_max - 1, nh, hd, pos_dev=pos_dev, workspace=ws)
    check(y3, want, dt, "fused decode attention, device-side position")
    y4 = pkg.hip.qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, cache, 1, B, pos0, nh, hd)
    check(y4, want, dt, "fused decode attention without workspace")
    # the single-launch variant for few (head, row) pairs: one 1024-thread workgroup each
    pkg.hip.set_tuning("attn_wide", 4096)
    try:
        y5 = pkg.hip.qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, cache, 1, B, pos0, nh, hd, workspace=ws)
    finally:
        pkg.hip.set_tuning("attn_wide", 0)
    check(y5, want, dt, "fused decode attention, one workgroup per head and row")
    assert torch.equal(kd, kd2) and torch.equal(vd, vd2)


@pytest.mark.parametrize("nh,hd,B,S,pos0,t_max,qscale", [
    (55, 96, 1, 512, 0, 1024, 1), (55, 96, 2, 100, 37, 1024, 1), (4, 64, 3, 64, 0, 1024, 1), (3, 128, 1, 65, 200, 1024, 1),
    (55, 96, 1, 2, 5, 1024, 1), (5, 96, 1, 300, 724, 1024, 1),
    # 128 query rows per workgroup (launches of 512 workgroups and more): ragged last block, a cache that ends inside the
    # last key tile, all three head sizes, and scores spread widely enough that the reference maximum moves (and O is
    # rescaled) in many tiles
    (55, 96, 2, 650, 300, 1024, 1), (16, 64, 4, 1000, 24, 1024, 1), (16, 128, 4, 900, 77, 1000, 1), (55, 96, 2, 640, 0, 640, 8),
    (55, 96, 1, 512, 0, 1024, 8)])
def test_prefill_attention_mfma(pkg, nh, hd, B, S, pos0, t_max, qscale):
    """The matrix-core chunk kernel against the oracle and against the per-row kernel."""
    dt = torch.bfloat16
    k, v, kd, vd, cache = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=130)
    q = (rnd((B * S, nh * hd), dt, 132) * qscale).to(dt)
    y = pkg.hip.prefill_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd)
    T = pos0 + S
    qq = q.view(B, S, nh, hd).transpose(1, 2)
    want = O.sdpa(qq, k[1, :, :, :T], v[1, :, :, :T]).transpose(1, 2).reshape(B * S, nh * hd)
    check(y, want, dt, f"prefill attention B={B} S={S} pos0={pos0}")
    y_rows = pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd)
    check(y, y_rows, dt, "chunk kernel vs per-row kernel")
    pos_dev = torch.tensor([pos0], dtype=torch.int32, device="cuda")
    y2 = pkg.hip.prefill_attention(q.cuda(), cache, 1, B, S, t_max - S, nh, hd, pos_dev=pos_dev)
    assert torch.equal(y2, y)
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.prefill_attention(q.float().cuda(), cache, 1, B, S, pos0, nh, hd)


def test_swiglu_elementwise(pkg):
    for dt, M, I in ((torch.bfloat16, 5, 17920), (torch.float32, 3, 704), (torch.bfloat16, 1, 8)):
        z = rnd((M, 2 * I), dt, 140)
        got = pkg.hip.swiglu(z.cuda())
        check(got, F.silu(z[:, :I]) * z[:, I:], dt, "swiglu", ulps=ULPS_SWIGLU)
        if dt == torch.bfloat16:
            assert bool((got.cpu() == F.silu(z[:, :I]) * z[:, I:]).float().mean() > 0.99)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_noise_mix_rounds_like_the_elementwise_expression_on_the_device(pkg, dt):
    """raven_noise_mix against the five forms of the state perturbation (recpre/raven_modeling_minimal.py:818-831)
    evaluated by torch on the GPU, where a 0-dim device tensor operand is converted to the result dtype first and a
    Python float is a float32 operand: bit-exact."""
    x, noise = rnd((3, 5280), dt, 160).cuda(), rnd((3, 5280), dt, 161).cuda()
    n = 0.3 * math.sqrt(0.4)
    f32 = lambda v: float(torch.tensor(v, dtype=torch.float32))
    st = lambda v: float(torch.tensor(v, dtype=torch.float32).to(dt))
    for step in (0, 2, 6):
        step1 = torch.as_tensor(step + 1, device="cuda")
        want = x * (1 - n / step1) + noise * n / step1
        got = pkg.hip.noise_mix(x, noise, st(1.0 - f32(f32(n) / (step + 1))), n, float(step + 1))
        assert torch.equal(got, want), f"geom, step {step}"
        root = step1.sqrt()
        want = x * (1 - n / root) + noise * n / root
        d32 = f32(math.sqrt(step + 1))
        got = pkg.hip.noise_mix(x, noise, st(1.0 - f32(f32(n) / d32)), n, st(d32))
        assert torch.equal(got, want), f"sqrt, step {step}"
        c = max(n, (8 - step) / 8)
        assert torch.equal(pkg.hip.noise_mix(x, noise, 1.0 - c, c), x * (1 - c) + noise * c), f"line, step {step}"
    assert torch.equal(pkg.hip.noise_mix(x, noise, 1.0 - n, n), x * (1 - n) + noise * n), "fixed"
    u = torch.tensor([0.3671875], device="cuda", dtype=dt)
    amp = 2 * u * n
    want = x * (1 - amp) + noise * amp
    c = st(st(2.0 * float(u)) * f32(n))
    assert torch.equal(pkg.hip.noise_mix(x, noise, st(1.0 - c), c), want), "chi"


def test_decode_attention_at_the_maximum_context(pkg):
    """block_size = 4096 positions (recpre/raven_config_minimal.py:17): the last decode step of a full context."""
    dt, nh, hd, t_max = torch.bfloat16, 55, 96, 4096
    k, v, kd, vd, cache = make_cache(pkg, 1, 1, nh, t_max, hd, dt, fill_seed=150)
    q = rnd((1, nh * hd), dt, 151)
    ws = pkg.hip.attention_workspace(1, nh, hd, "cuda")
    y = pkg.hip.decode_attention(q.cuda(), cache, 0, 1, 1, t_max - 1, nh, hd, workspace=ws)
    want = O.sdpa(q.view(1, 1, nh, hd).transpose(1, 2), k[0], v[0]).transpose(1, 2).reshape(1, nh * hd)
    check(y, want, dt, "attention over 4096 positions")
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.decode_attention(q.cuda(), cache, 0, 1, 1, t_max, nh, hd, workspace=ws)  # one past the end


@pytest.mark.parametrize("B,S,pos0", [(1, 1, 1000), (32, 1, 300), (2, 3, 200)])
@pytest.mark.parametrize("mode", ["skip", "latest", "always_last"])
def test_decode_attention_partially_filled_slots(pkg, mode, B, S, pos0):
    """steps_present: positions of earlier tokens hold different numbers of core steps; the kernel reads each from the
    slot the lookup rule names (or leaves it out) -- checked against a gather done on the host, at the 3.5b head shape,
    with and without the split over positions, unfused and fused."""
    dt, nh, hd, t_max, h = torch.bfloat16, 55, 96, 1024, 55 * 96
    n_slots, core0 = 14, 2          # slots 0, 1: coda; 2..13: core steps 0..11 (three recurrences of four blocks)
    k, v = rnd((n_slots, B, nh, t_max, hd), dt, 200), rnd((n_slots, B, nh, t_max, hd), dt, 201)
    kd, vd = k.cuda(), v.cuda()
    g = torch.Generator().manual_seed(202)
    depth = torch.randint(1, 4, (t_max,), generator=g, dtype=torch.int32) * 4  # 4, 8 or 12 core steps per position
    code = {"skip": pkg.hip.LOOKUP_SKIP, "latest": pkg.hip.LOOKUP_LATEST, "always_last": pkg.hip.LOOKUP_ALWAYS_LAST}[mode]
    depth_d = depth.cuda()          # the descriptor holds raw pointers: keep the tensors alive
    cache = pkg.hip.make_cache(kd, vd, depth_d, code, core0)
    ws = pkg.hip.attention_workspace(B * S, nh, hd, "cuda")
    T = pos0 + S
    for cs in (1, 6, 11):           # the step being read: first, second, third recurrence
        slot = core0 + cs
        src = torch.full((T,), slot, dtype=torch.long)
        keep = torch.ones(T, dtype=torch.bool)
        for p in range(pos0):       # positions from pos0 on are the call's own rows
            d, j = int(depth[p]), cs % 4
            if mode != "always_last" and cs < d:
                continue
            if mode == "skip":
                keep[p] = False
            else:
                src[p] = core0 + j + (d - 1 - j) // 4 * 4
        ar = torch.arange(T)
        kk, vv = k[src, :, :, ar].permute(1, 2, 0, 3), v[src, :, :, ar].permute(1, 2, 0, 3)  # [B, nh, T, hd]
        q = rnd((B * S, h), dt, 203 + cs)
        qq = q.view(B, S, nh, hd).transpose(1, 2).float()
        mask = keep.view(1, T).expand(S, T) & torch.ones(S, T, dtype=torch.bool).tril(T - S)
        want = F.scaled_dot_product_attention(qq, kk.float(), vv.float(), attn_mask=mask).transpose(1, 2).reshape(B * S, h)
        y = pkg.hip.decode_attention(q.cuda(), cache, slot, B, S, pos0, nh, hd, workspace=ws)
        check(y, want, dt, f"{mode} cs={cs}")
        y = pkg.hip.decode_attention(q.cuda(), cache, slot, B, S, pos0, nh, hd)
        check(y, want, dt, f"{mode} cs={cs}, no split")
    # the fused decode step appends its own row and resolves the older ones the same way
    if S == 1:
        cs, slot = 6, core0 + 6
        qkv = rnd((B, 3 * h), dt, 210)
        table = O.rope_table(hd, t_max, 50000.0).to(dt)
        freqs = table.float().reshape(t_max, hd // 2, 2).contiguous().cuda()
        kd2, vd2 = kd.clone(), vd.clone()
        c2 = pkg.hip.make_cache(kd2, vd2, depth_d, code, core0)
        y_f = pkg.hip.qkv_attention_decode(qkv.cuda(), None, freqs, cache, slot, B, pos0, nh, hd, workspace=ws)
        q2 = pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), None, freqs, c2, slot, B, 1, pos0, nh, hd)
        y_2 = pkg.hip.decode_attention(q2, c2, slot, B, 1, pos0, nh, hd, workspace=ws)
        assert torch.equal(kd, kd2) and torch.equal(vd, vd2)
        check(y_f, y_2.float().cpu(), dt, f"{mode}: fused equals append-then-attend")
    # prelude / coda slots ignore the lookup table
    q = rnd((B * S, h), dt, 220)
    plain = pkg.hip.make_cache(kd, vd)
    assert torch.equal(pkg.hip.decode_attention(q.cuda(), cache, 0, B, S, pos0, nh, hd, workspace=ws),
                       pkg.hip.decode_attention(q.cuda(), plain, 0, B, S, pos0, nh, hd, workspace=ws))
    with pytest.raises(pkg.hip.RavenHipError, match="steps_present"):
        pkg.hip.prefill_attention(q.cuda(), cache, core0, B, S, pos0, nh, hd)


def test_decode_attention_zero_query_gives_mean(pkg):
    dt, nh, hd, T = torch.bfloat16, 55, 96, 513
    k, v, kd, vd, cache = make_cache(pkg, 1, 1, nh, 1024, hd, dt, fill_seed=95)
    y = pkg.hip.decode_attention(torch.zeros(1, nh * hd, dtype=dt, device="cuda"), cache, 0, 1, 1, T - 1, nh, hd)
    check(y.view(nh, hd), v[0, 0, :, :T].float().mean(1), dt, "q=0 -> mean of V")


# ----------------------------------------------------------------------------- embed / argmax
def test_embed_and_argmax(pkg):
    for dt in (torch.bfloat16, torch.float32):
        wte = rnd((1000, 256), dt, 100, 0.02)
        ids = torch.tensor([0, 999, 17, 17, 500])
        got = pkg.hip.embed(wte.cuda(), ids.cuda(), 16.0)
        assert torch.equal(got.cpu(), F.embedding(ids, wte) * 16.0)
        got = pkg.hip.embed(wte.cuda(), ids.cuda(), math.sqrt(5280))
        assert torch.equal(got.cpu(), F.embedding(ids, wte) * math.sqrt(5280))
    logits = rnd((5, 65536), torch.float32, 101)
    logits[1, 7] = logits[1, 60000] = 99.0      # tie: the first index wins
    logits[2, 65535] = 100.0
    logits[3] = -float("inf")
    assert torch.equal(pkg.hip.argmax(logits.cuda()).cpu(), logits.argmax(-1))
    small = rnd((3, 1024), torch.float32, 102)
    assert torch.equal(pkg.hip.argmax(small.cuda()).cpu(), small.argmax(-1))


# ----------------------------------------------------------------------------- adaptive-compute exit statistics
@pytest.mark.parametrize("B,V", [(1, 65536), (3, 65536), (32, 1024), (2, 1000)])
def test_exit_logit_stats(pkg, B, V):
    """Entropy, KL and min-p KL of successive logits rows against the oracle's evaluators (fp32; sums over V terms
    in another order: absolute 2e-5 + relative 1e-4)."""
    g = torch.Generator().manual_seed(300 + B)
    steps = [torch.randn(B, V, generator=g) * 3 for _ in range(2)]
    steps.append(steps[-1] + torch.randn(B, V, generator=g) * 1e-2)     # a small change: KL of the order 1e-4
    steps.append(steps[-1].clone())                                     # no change: KL 0
    fake = lambda lg: (lambda lat: O.OracleOutput(logits=lg.unsqueeze(1), latent_states=lat))
    lat = torch.zeros(B, 1, 4)
    for kind, code in (("entropy-diff", pkg.hip.EXIT_ENTROPY), ("kl", pkg.hip.EXIT_KL), ("minp-kl", pkg.hip.EXIT_MINP_KL)):
        ev = O.ExitCriterion(kind, "auto", V)
        ev.init(lat)
        prev = ((1 / V) * torch.ones(B, V)).log().cuda()
        for i, lg in enumerate(steps):
            ev.check(lat, fake(lg))
            got = pkg.hip.exit_logit_stats(lg.cuda(), code, None if kind == "entropy-diff" else prev)
            want = ev.prev if kind == "entropy-diff" else None
            if kind == "entropy-diff":
                assert torch.allclose(got.cpu(), want, rtol=1e-4, atol=2e-5), (kind, i, got, want)
            else:
                break
        # KL kinds: compare the values and the stored log-probabilities step by step
        if kind != "entropy-diff":
            ev.init(lat)
            prev = ((1 / V) * torch.ones(B, V)).log().cuda()
            for i, lg in enumerate(steps):
                _, _, v = ev.check(lat, fake(lg))
                got = pkg.hip.exit_logit_stats(lg.cuda(), code, prev)
                assert torch.allclose(got.cpu(), v, rtol=1e-3, atol=2e-5), (kind, i, got, v)
                assert torch.allclose(prev.cpu(), ev.prev, rtol=1e-5, atol=1e-5), (kind, i)
            assert float(got.abs().max()) < 1e-6                        # identical successive rows
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.exit_logit_stats(steps[0].cuda(), pkg.hip.EXIT_KL)      # KL without the previous log-probabilities


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_exit_latent_stats(pkg, dt):
    B, S, h = 3, 5, 5280
    a, b = rnd((B, S, h), dt, 310), rnd((B, S, h), dt, 311)
    b = (a.float() * 0.9 + b.float() * 0.3).to(dt)
    rel, cos = pkg.hip.exit_latent_stats(a.view(-1, h).cuda(), b.view(-1, h).cuda(), want_rel=True, want_cos=True)
    want_rel = (a - b).norm(dim=-1) / a.norm(dim=-1)                     # the reference's expressions, in dtype
    want_cos = (a * b).sum(dim=-1) / a.norm(dim=-1) / b.norm(dim=-1)
    tol = dict(rtol=2e-2, atol=1e-2) if dt == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
    assert rel.dtype == dt and torch.allclose(rel.float().cpu().view(B, S), want_rel.float(), **tol)
    assert torch.allclose(cos.float().cpu().view(B, S), want_cos.float(), **tol)
    # closed forms: a = 2 b -> 1/2 and cosine 1; orthogonal rows -> cosine 0
    x = torch.zeros(2, h, dtype=dt)
    x[0, :7], x[1, 0] = 1.0, 3.0
    y = x.clone() * 0.5
    y[1] = 0
    y[1, 1] = 2.0
    rel, cos = pkg.hip.exit_latent_stats(x.cuda(), y.cuda(), want_rel=True, want_cos=True)
    assert abs(float(rel[0]) - 0.5) < 1e-6 and abs(float(cos[0]) - 1.0) < 1e-2 and float(cos[1]) == 0.0


# ----------------------------------------------------------------------------- fp32 at the 3.5b shape
def test_fp32_kernels_at_the_3_5b_shape(pkg):
    """The reference runs in fp32 at any shape; the fp32 variants here need more registers / LDS per row at h = 5280,
    hd = 96, I = 17920: rows of 1320 chunks for the norm, 24 chunks per head row (two per lane) for attention, X rows
    of up to 71680 bytes in the vector GEMM's LDS."""
    dt, h, nh, hd, I = torch.float32, 5280, 55, 96, 17920
    x, res, w = rnd((3, h), dt, 400), rnd((3, h), dt, 401), 1 + rnd((h,), dt, 402, 0.02)
    y, _, _ = pkg.hip.rmsnorm_residual(x.cuda(), w.cuda(), 1e-6, residual=res.cuda())
    check(y, O.rmsnorm(x + res, w, 1e-6), dt, "rmsnorm fp32 5280")
    for M in (1, 3, 8):
        xi, wm = rnd((M, I), dt, 403 + M), rnd((256, I), dt, 404, 0.02)
        check(pkg.hip.gemm(xi.cuda(), wm.cuda()), lin(xi, wm), dt, f"fp32 gemm K=17920 M={M}")
        xa, wa = rnd((M, 2 * h), dt, 405 + M), rnd((128, 2 * h), dt, 406, 0.02)
        check(pkg.hip.gemm(xa.cuda(), wa.cuda()), lin(xa, wa), dt, f"fp32 gemm K=10560 M={M}")
    # attention: decode step (fused and two-step), a chunk of rows, with and without the split over positions
    t_max, B = 300, 2
    k, v, kd, vd, cache = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=410)
    ws = pkg.hip.attention_workspace(B * 3, nh, hd, "cuda")
    for S, pos0 in ((1, 200), (3, 100), (1, 0)):
        q = rnd((B * S, nh * hd), dt, 412 + S)
        T = pos0 + S
        want = O.sdpa(q.view(B, S, nh, hd).transpose(1, 2), k[1, :, :, :T], v[1, :, :, :T]).transpose(1, 2).reshape(B * S, nh * hd)
        check(pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd, workspace=ws), want, dt, f"fp32 hd=96 attention S={S}")
        check(pkg.hip.decode_attention(q.cuda(), cache, 1, B, S, pos0, nh, hd), want, dt, f"fp32 hd=96 attention S={S}, no split")
    qkv, bias = rnd((B, 3 * nh * hd), dt, 420), rnd((2, 1, nh, hd), dt, 421, 0.5)
    table = O.rope_table(hd, t_max, 50000.0)
    freqs = table.reshape(t_max, hd // 2, 2).contiguous().cuda()
    k2, v2, kd2, vd2, cache2 = make_cache(pkg, 2, B, nh, t_max, hd, dt, fill_seed=410)
    y_f = pkg.hip.qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, cache, 1, B, 150, nh, hd, workspace=ws)
    q2 = pkg.hip.qkv_bias_rope_cache_append(qkv.cuda(), bias.cuda(), freqs, cache2, 1, B, 1, 150, nh, hd)
    y_2 = pkg.hip.decode_attention(q2, cache2, 1, B, 1, 150, nh, hd, workspace=ws)
    assert torch.equal(kd, kd2) and torch.equal(vd, vd2)
    check(y_f, y_2.cpu(), dt, "fp32 hd=96 fused decode step")


# ----------------------------------------------------------------------------- paged KV cache (vLLM layout)
@pytest.mark.parametrize("dt,nh,hd,B,block_size,layout", [(torch.bfloat16, 55, 96, 1, 16, "NHD"), (torch.bfloat16, 55, 96, 32, 16, "NHD"),
                                                          (torch.bfloat16, 55, 96, 5, 32, "HND"), (torch.float32, 4, 64, 3, 8, "NHD"),
                                                          (torch.float32, 5, 96, 2, 16, "HND"), (torch.bfloat16, 55, 96, 32, 16, "HND"),
                                                          (torch.bfloat16, 4, 64, 3, 12, "HND"), (torch.bfloat16, 4, 64, 3, 12, "NHD")])
def test_paged_decode_attention_and_append(pkg, dt, nh, hd, B, block_size, layout):
    """Block-paged K/V with shuffled block tables and a different length per sequence (1 and 0 among them): appended rows
    land in their slots, attention equals torch SDPA per sequence, and -- for equal lengths -- the contiguous kernel's bits.
    Both page layouts ([blocks, block_size, heads, hd] and [blocks, heads, block_size, hd]); a block size that is no power of two."""
    h = nh * hd
    lay = pkg.hip.PAGED_NHD if layout == "NHD" else pkg.hip.PAGED_HND
    rows_of = (lambda c: c.view(-1, nh, hd)) if layout == "NHD" else (lambda c: c.permute(0, 2, 1, 3).reshape(-1, nh, hd))
    g = torch.Generator().manual_seed(600 + B)
    max_len = 700
    max_blocks = (max_len + block_size - 1) // block_size
    num_blocks = B * max_blocks + 3
    lens = torch.randint(2, max_len + 1, (B,), generator=g, dtype=torch.int32)
    lens[0] = max_len
    if B > 2:
        lens[1], lens[2] = 1, 0
    table = torch.randperm(num_blocks, generator=g)[:B * max_blocks].view(B, max_blocks).to(torch.int32)
    k_seq, v_seq = rnd((B, max_len, nh, hd), dt, 601), rnd((B, max_len, nh, hd), dt, 602)
    kc = torch.zeros((num_blocks, block_size, nh, hd) if layout == "NHD" else (num_blocks, nh, block_size, hd), dtype=dt, device="cuda")
    vc = torch.zeros_like(kc)
    # fill the cache through the append kernel: every sequence's positions, in one call, plus a skipped row
    rows_k, rows_v, slots = [], [], []
    for b in range(B):
        for p in range(int(lens[b])):
            rows_k.append(k_seq[b, p].reshape(-1))
            rows_v.append(v_seq[b, p].reshape(-1))
            slots.append(int(table[b, p // block_size]) * block_size + p % block_size)
    rows_k.append(torch.ones(h, dtype=dt))
    rows_v.append(torch.ones(h, dtype=dt))
    slots.append(-1)
    kk, vv, sl = torch.stack(rows_k).cuda(), torch.stack(rows_v).cuda(), torch.tensor(slots, dtype=torch.int64).cuda()
    for lo in range(0, kk.shape[0], 60000):
        pkg.hip.paged_kv_append(kk[lo:lo + 60000].contiguous(), vv[lo:lo + 60000].contiguous(), kc, vc, sl[lo:lo + 60000].contiguous(),
                                layout=lay)
    flat_k = rows_of(kc).cpu()
    for b in range(B):
        for p in (0, int(lens[b]) - 1):
            if p >= 0 and int(lens[b]) > 0:
                assert torch.equal(flat_k[int(table[b, p // block_size]) * block_size + p % block_size], k_seq[b, p])
    assert int((flat_k.abs().amax(dim=(1, 2)) > 0).sum()) == int(lens.sum())  # nothing written anywhere else (the -1 row is skipped)
    q = rnd((B, h), dt, 603)
    ws = pkg.hip.attention_workspace(B, nh, hd, "cuda")
    for wsp in (ws, None):
        y = pkg.hip.paged_decode_attention(q.cuda(), kc, vc, table.cuda(), lens.cuda(), max_len, workspace=wsp, layout=lay)
        for b in range(B):
            n = int(lens[b])
            if n == 0:
                assert float(y[b].abs().max()) == 0.0
                continue
            want = F.scaled_dot_product_attention(q[b].view(1, nh, 1, hd).float(), k_seq[b, :n].transpose(0, 1).unsqueeze(0).float(),
                                                  v_seq[b, :n].transpose(0, 1).unsqueeze(0).float()).reshape(h)
            check(y[b], want, dt, f"paged attention, sequence {b} of length {n}")
    # equal lengths: the same numbers as the contiguous cache kernel gives (same arithmetic, other addresses)
    n = 300
    eq = torch.full((B,), n, dtype=torch.int32)
    y = pkg.hip.paged_decode_attention(q.cuda(), kc, vc, table.cuda(), eq.cuda(), n, layout=lay)
    kd = torch.zeros(1, B, nh, n, hd, dtype=dt)
    vd = torch.zeros_like(kd)
    for b in range(B):
        m = min(n, int(lens[b]))
        kd[0, b, :, :m], vd[0, b, :, :m] = k_seq[b, :m].transpose(0, 1), v_seq[b, :m].transpose(0, 1)
    kdd, vdd = kd.cuda(), vd.cuda()
    want = pkg.hip.decode_attention(q.cuda(), pkg.hip.make_cache(kdd, vdd), 0, B, 1, n - 1, nh, hd)
    full = [b for b in range(B) if int(lens[b]) >= n]
    check(y[full], want[full].float().cpu(), dt, "paged vs contiguous")
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.paged_decode_attention(q.cuda(), kc, vc, table.cuda(), lens.cuda(), max_blocks * block_size + 1, layout=lay)

    # The fused decode step: sequence b's new token at position lens[b] - 1 (its page currently holds k_seq / v_seq of
    # that position, which the step overwrites).  Against the oracle's bias + RoPE per sequence, the append kernel and
    # the attention kernel above -- same results, and the same cache afterwards.
    qkv = rnd((B, 3 * h), dt, 604)
    bias = rnd((2, nh, hd), dt, 605, 0.5)
    rope = O.rope_table(hd, max_len, 50000.0).to(dt)
    freqs = rope.float().reshape(max_len, hd // 2, 2).contiguous().cuda()
    kc2, vc2 = kc.clone(), vc.clone()
    for wsp in (ws, None):
        y_f = pkg.hip.paged_qkv_attention_decode(qkv.cuda(), bias.cuda(), freqs, kc, vc, table.cuda(), lens.cuda(), max_len, workspace=wsp,
                                                 layout=lay)
    rows_q, rows_k, rows_v, slots = [], [], [], []
    for b in range(B):
        n = int(lens[b])
        qq, kk, vv = (t.view(1, 1, nh, hd) for t in qkv[b].split([h, h, h]))
        if n == 0:
            rows_q.append(torch.zeros(h, dtype=dt)); rows_k.append(torch.zeros(h, dtype=dt)); rows_v.append(torch.zeros(h, dtype=dt))
            slots.append(-1)
            continue
        qq, kk = (qq + bias[0]).to(dt), (kk + bias[1]).to(dt)
        rq, rk = O.apply_rope(qq, kk, rope[:, n - 1:n])
        rows_q.append(rq.reshape(h)); rows_k.append(rk.reshape(h)); rows_v.append(vv.reshape(h))
        slots.append(int(table[b, (n - 1) // block_size]) * block_size + (n - 1) % block_size)
    pkg.hip.paged_kv_append(torch.stack(rows_k).cuda(), torch.stack(rows_v).cuda(), kc2, vc2, torch.tensor(slots, dtype=torch.int64).cuda(),
                            layout=lay)
    y_2 = pkg.hip.paged_decode_attention(torch.stack(rows_q).cuda(), kc2, vc2, table.cuda(), lens.cuda(), max_len, workspace=ws, layout=lay)
    check(y_f, y_2.float().cpu(), dt, "fused paged step vs rope + append + attention")
    check(kc, kc2.float().cpu(), dt, "keys after the fused paged step")
    assert torch.equal(vc, vc2)
    assert int((rows_of(kc).abs().amax(dim=(1, 2)) > 0).sum()) == int(lens.sum())  # no other row was touched


@pytest.mark.parametrize("nh,hd,block_size,layout,chunks", [
    (55, 96, 16, "HND", ((0, 300), (212, 40), (699, 1), (0, 0), (64, 64), (5, 130))),
    (55, 96, 16, "NHD", ((0, 200), (100, 100))),
    (4, 64, 12, "HND", ((0, 77), (30, 300))),
    (3, 128, 32, "NHD", ((1, 129), (500, 200), (0, 1))),
    (55, 96, 16, "HND", tuple((37 * i % 200, 640) for i in range(10))),   # 128-row workgroups
])
def test_paged_rope_append_and_prefill_attention_of_several_sequences(pkg, nh, hd, block_size, layout, chunks):
    """Prompt chunks and decode rows of several sequences in one launch each, over shuffled pages: chunk (context, rows)
    means the sequence already holds `context` positions and `rows` new ones arrive.  raven_paged_qkv_rope_append against
    the oracle's bias + RoPE per row (and the slots it must fill), raven_paged_prefill_attention against torch SDPA with a
    lower-right aligned causal mask per sequence, and against the contiguous-cache kernel's bits."""
    dt, h = torch.bfloat16, nh * hd
    lay = pkg.hip.PAGED_NHD if layout == "NHD" else pkg.hip.PAGED_HND
    B = len(chunks)
    g = torch.Generator().manual_seed(700 + B + block_size)
    max_len = max(c + r for c, r in chunks) + 3
    max_blocks = (max_len + block_size - 1) // block_size
    num_blocks = B * max_blocks + 2
    table = torch.randperm(num_blocks, generator=g)[:B * max_blocks].view(B, max_blocks).to(torch.int32)
    shape = (num_blocks, block_size, nh, hd) if layout == "NHD" else (num_blocks, nh, block_size, hd)
    kc, vc = torch.zeros(shape, dtype=dt, device="cuda"), torch.zeros(shape, dtype=dt, device="cuda")
    slot_of = lambda b, p: int(table[b, p // block_size]) * block_size + p % block_size
    # the contexts: already rotated keys, through the plain append kernel
    k_ctx = [rnd((c, nh, hd), dt, 710 + b) for b, (c, r) in enumerate(chunks)]
    v_ctx = [rnd((c, nh, hd), dt, 740 + b) for b, (c, r) in enumerate(chunks)]
    rows = [(b, p) for b, (c, r) in enumerate(chunks) for p in range(c)]
    if rows:
        pkg.hip.paged_kv_append(torch.stack([k_ctx[b][p].reshape(-1) for b, p in rows]).cuda(),
                                torch.stack([v_ctx[b][p].reshape(-1) for b, p in rows]).cuda(), kc, vc,
                                torch.tensor([slot_of(b, p) for b, p in rows], dtype=torch.int64).cuda(), layout=lay)
    # the new rows of all sequences, flattened as a serving engine hands them over, plus one row that is not stored
    T = sum(r for c, r in chunks)
    qkv = rnd((T + 1, 3 * h), dt, 770)
    bias = rnd((2, nh, hd), dt, 771, 0.5)
    rope = O.rope_table(hd, max_len, 50000.0).to(dt)
    freqs = rope.float().reshape(max_len, hd // 2, 2).contiguous().cuda()
    positions = torch.tensor([c + i for c, r in chunks for i in range(r)] + [0], dtype=torch.int64)
    slots = torch.tensor([slot_of(b, c + i) for b, (c, r) in enumerate(chunks) for i in range(r)] + [-1], dtype=torch.int64)
    before = kc.clone()
    q = pkg.hip.paged_qkv_rope_append(qkv.cuda(), bias.cuda(), freqs, positions.cuda(), slots.cuda(), kc, vc, layout=lay)
    qq, kk, vv = (t.view(T + 1, 1, nh, hd) for t in qkv.split([h, h, h], dim=1))
    qq, kk = (qq + bias[0]).to(dt), (kk + bias[1]).to(dt)
    want_q, want_k = torch.empty(T + 1, nh, hd, dtype=dt), torch.empty(T + 1, nh, hd, dtype=dt)
    for t in range(T + 1):
        rq, rk = O.apply_rope(qq[t:t + 1], kk[t:t + 1], rope[:, int(positions[t]):int(positions[t]) + 1])
        want_q[t], want_k[t] = rq.view(nh, hd), rk.view(nh, hd)
    assert torch.equal(q.cpu().view(T + 1, nh, hd), want_q)
    rows_of = (lambda c: c.view(-1, nh, hd)) if layout == "NHD" else (lambda c: c.permute(0, 2, 1, 3).reshape(-1, nh, hd))
    flat_k, flat_v = rows_of(kc).cpu(), rows_of(vc).cpu()
    for t in range(T):
        assert torch.equal(flat_k[int(slots[t])], want_k[t]) and torch.equal(flat_v[int(slots[t])], vv[t, 0])
    untouched = torch.ones(flat_k.shape[0], dtype=torch.bool)
    untouched[slots[:T]] = False
    assert torch.equal(flat_k[untouched], rows_of(before).cpu()[untouched])  # the row with slot -1 went nowhere

    lens = torch.tensor([c + r for c, r in chunks], dtype=torch.int32)
    q_start = torch.tensor([0] + list(torch.tensor([r for c, r in chunks]).cumsum(0)), dtype=torch.int32)
    max_q = max(r for c, r in chunks)
    y = pkg.hip.paged_prefill_attention(q[:T].contiguous(), kc, vc, table.cuda(), lens.cuda(), q_start.cuda(), max_q, layout=lay)
    t0 = 0
    for b, (c, r) in enumerate(chunks):
        if r == 0:
            continue
        keys = torch.cat([k_ctx[b], want_k[t0:t0 + r]]).transpose(0, 1).unsqueeze(0)      # [1, nh, c + r, hd]
        vals = torch.cat([v_ctx[b], vv[t0:t0 + r, 0]]).transpose(0, 1).unsqueeze(0)
        want = O.sdpa(want_q[t0:t0 + r].transpose(0, 1).unsqueeze(0), keys, vals).transpose(1, 2).reshape(r, h)
        check(y[t0:t0 + r], want, dt, f"paged prefill attention, sequence {b}: {r} rows after {c}")
        if r >= 2:   # the contiguous-cache kernel on the same keys: same arithmetic, other addresses
            kd, vd = keys.unsqueeze(0).contiguous().cuda(), vals.unsqueeze(0).contiguous().cuda()
            same = pkg.hip.prefill_attention(q[t0:t0 + r].contiguous(), pkg.hip.make_cache(kd, vd), 0, 1, r, c, nh, hd)
            if (max_q + 127) // 128 * nh * B >= 512 and (r + 127) // 128 * nh < 512:
                check(y[t0:t0 + r], same, dt, "paged vs contiguous (other rows per workgroup)")
            else:
                assert torch.equal(y[t0:t0 + r], same), f"paged vs contiguous, sequence {b}"
        t0 += r
    with pytest.raises(pkg.hip.RavenHipError):
        pkg.hip.paged_prefill_attention(q[:T].float(), kc.float(), vc.float(), table.cuda(), lens.cuda(), q_start.cuda(), max_q, layout=lay)
