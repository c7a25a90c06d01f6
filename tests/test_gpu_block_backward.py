"""The backward pass of the Mamba-2 block's stages through the C ABI (ssd_block_post_bwd, ssd_block_pre_bwd) against
the float64 oracle, whose gradients are pinned by central differences in tests/test_oracle_block.py, and of the whole
block (Mamba2Block.backward: GEMMs + post, scan and pre backward) against the oracle's block gradients.

Bars.  float32: max|err| / rms <= 1e-4 for activation gradients; parameter gradients, sums over batch and time of
terms of either sign, on the scale of the summed terms' 2-norm (the way the scan's dA and dD are judged).  bf16:
activation gradients are stored in bf16, so each element is allowed one bf16 rounding of itself (2^-8 |ref|) on top
of 2e-2 rms; parameter gradients (float32 sums of products of bf16-rounded factors) 2e-2 on the 2-norm scale.  The
reference holds no backward of this layer, so parity with it is unpinned by the reference."""
import numpy as np
import pytest
import torch

from oracle import mamba2_block_oracle as blk
from trading_bot_0_amd import Mamba2Block, block_post, block_post_bwd, block_pre_bwd

from _util import np64

pytestmark = pytest.mark.gpu


def params(H, P, N, G, K, seed=0):
    g = torch.Generator().manual_seed(seed)
    C = H * P + 2 * G * N
    return dict(conv_w=torch.randn(C, K, generator=g).cuda() / 2, conv_b=torch.randn(C, generator=g).cuda() / 4,
                dt_bias=torch.randn(H, generator=g).cuda(), norm_w=torch.randn(H * P, generator=g).cuda())


def check_act(out, ref, dtype, what):
    o = out.detach().float().cpu().numpy().astype(np.float64).reshape(ref.shape)
    rms = float(np.sqrt(np.mean(ref * ref)))
    assert np.isfinite(o).all(), what
    if rms == 0.0:  # an all-zero reference (a gradient cut off by a restart): exactly zero
        assert not o.any(), f"{what}: the reference is zero, the output is not"
    elif dtype == torch.float32:
        e = np.abs(o - ref).max() / rms
        assert e <= 1e-4, f"{what}: {e:.3e}"
    else:
        over = np.abs(o - ref) - (2e-2 * rms + 2.0 ** -8 * np.abs(ref))
        assert over.max() <= 0, f"{what}: exceeds 2e-2 rms + 2^-8 |ref| by {over.max():.3e} (rms {rms:.3e})"


def check_sum(out, ref, scale, dtype, what):
    """A parameter gradient against its reference on the scale of the 2-norm of the terms it sums."""
    o = out.detach().float().cpu().numpy().astype(np.float64).reshape(ref.shape)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    e = (np.abs(o - ref) / np.maximum(scale, 1e-30)).max()
    assert np.isfinite(o).all() and e <= tol, f"{what}: {e:.3e} of the summed terms' 2-norm"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1), (3, 7, 8, 16, 16, 2), (1, 33, 16, 64, 128, 2), (5, 300, 8, 32, 64, 1),
                                   (2, 9, 8, 24, 16, 1), (1, 21, 24, 24, 16, 1), (3, 70, 40, 40, 16, 1)])  # rows the lanes do not cover exactly
def test_post_backward(shape, dtype):
    Bsz, L, H, P, N, G = shape
    p = params(H, P, N, G, 4)
    g = torch.Generator().manual_seed(21)
    E = 2 * H * P + 2 * G * N + H
    z = torch.randn(Bsz, L, E, generator=g).to(dtype).cuda()
    y = (torch.randn(Bsz, L, H, P, generator=g) * 2).to(dtype).cuda()
    dout = torch.randn(Bsz, L, H * P, generator=g).to(dtype).cuda()
    dzx = torch.full_like(z, float("nan"))
    dy, dw = block_post_bwd(y, z, p["norm_w"], dout, dzx, H, P, N, G)
    torch.cuda.synchronize()
    ry, rz, rw = blk.block_post_bwd(np64(y), np64(z), np64(p["norm_w"]), 1e-5, np64(dout))
    check_act(dy, ry, dtype, "dy")
    check_act(dzx[..., :H * P], rz, dtype, "dz")
    assert torch.isnan(dzx[..., H * P:].float()).all(), "post_bwd writes only the z channels"
    # dnorm_w[c] sums dout * v * r over the rows
    yv, zv = np64(y).reshape(Bsz, L, -1), np64(z)[..., :H * P]
    v = yv * blk.silu(zv)
    r = 1.0 / np.sqrt((v * v).mean(-1, keepdims=True) + 1e-5)
    scale = np.sqrt(((np64(dout) * v * r) ** 2).sum((0, 1)))
    check_sum(dw, rw, scale, dtype, "dnorm_w")
    # the same bits on a second run (fixed summation order)
    dzx2 = torch.empty_like(z)
    dy2, dw2 = block_post_bwd(y, z, p["norm_w"], dout, dzx2, H, P, N, G)
    assert torch.equal(dw, dw2) and torch.equal(dy, dy2)
    # with yn_out, the forward's normalised rows on the way (for a forward that ran gate, norm and out-projection as
    # one kernel and kept none): bit for bit what block_post writes, the gradients unchanged
    yn = torch.full((Bsz, L, H * P), float("nan"), dtype=dtype, device="cuda")
    dy4, dw4 = block_post_bwd(y, z, p["norm_w"], dout, dzx2, H, P, N, G, yn_out=yn)
    assert torch.equal(yn, block_post(y, z, p["norm_w"], H, P, N, G)), "yn_out is not block_post's output"
    assert torch.equal(dy4, dy) and torch.equal(dw4, dw)
    if dtype == torch.bfloat16:   # the scan's float32 y as the forward's input
        y32 = y.float() + 1e-3
        dy3, dw3 = block_post_bwd(y32, z, p["norm_w"], dout, dzx2, H, P, N, G, yn_out=yn)
        ry3, _, rw3 = blk.block_post_bwd(np64(y32), np64(z), np64(p["norm_w"]), 1e-5, np64(dout))
        check_act(dy3, ry3, dtype, "dy from float32 y")
        check_sum(dw3, rw3, scale, dtype, "dnorm_w from float32 y")
        assert torch.equal(yn, block_post(y32, z, p["norm_w"], H, P, N, G)), "yn_out from float32 y"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1, 4), (3, 19, 8, 16, 16, 2, 3), (2, 33, 8, 32, 32, 1, 2),
                                   (3, 2, 8, 32, 64, 1, 4), (4, 1, 8, 32, 64, 1, 4), (2, 300, 16, 64, 128, 2, 4)])
def test_pre_backward(shape, dtype):
    """With and without a carried conv state, restarts (both sides of the kernel's runs of 32 steps, back to back, first
    and last step) and a gradient on the returned conv state."""
    Bsz, L, H, P, N, G, K = shape
    p = params(H, P, N, G, K)
    C = H * P + 2 * G * N
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(22)
    z = torch.randn(Bsz, L, E, generator=g).to(dtype).cuda()
    st = torch.randn(Bsz, K - 1, C, generator=g).to(dtype).cuda()
    dx = torch.randn(Bsz, L, H, P, generator=g).to(dtype).cuda()
    dB = torch.randn(Bsz, L, G, N, generator=g).to(dtype).cuda()
    dC = torch.randn(Bsz, L, G, N, generator=g).to(dtype).cuda()
    ddt = torch.randn(Bsz, L, H, generator=g).to(dtype).cuda()
    dso = torch.randn(Bsz, K - 1, C, generator=g).to(dtype).cuda()
    reset = torch.zeros(Bsz, L, dtype=torch.uint8)
    for t in (0, 5, 6, 15, 16, 17, 30, 31, 32, 33, 34, 63, 64, 65, 66, L - 1):
        if 0 <= t < L:
            reset[t % Bsz, t] = 1
    for state, rs, gso in ((None, None, None), (st, None, dso), (st, reset, dso), (None, reset, None)):
        dzx = torch.full_like(z, float("nan"))
        dcw, dcb, ddb, dst = block_pre_bwd(z, p["conv_w"], p["conv_b"], p["dt_bias"], dx, dB, dC, ddt, dzx, H, P, N, G,
                                           conv_state=state, reset=None if rs is None else rs.cuda(), dconv_state_out=gso,
                                           need_dconv_state=True)
        torch.cuda.synchronize()
        ref = blk.block_pre_bwd(np64(z), np64(p["conv_w"]), np64(p["conv_b"]), np64(p["dt_bias"]), H, P, N, G, np64(dx),
                                np64(dB), np64(dC), np64(ddt), None if state is None else np64(state),
                                None if rs is None else rs.numpy(), None if gso is None else np64(gso))
        tag = f"state={state is not None} reset={rs is not None}"
        check_act(dzx[..., H * P:H * P + C], ref[0], dtype, f"dxbc {tag}")
        check_act(dzx[..., H * P + C:], ref[1], dtype, f"ddt_raw {tag}")
        assert torch.isnan(dzx[..., :H * P].float()).all(), "pre_bwd leaves the z channels alone"
        check_act(dst, ref[5], dtype, f"dconv_state {tag}")
        # scales of the parameter sums: 2-norms of their terms, from the oracle's pieces
        zz = np64(z)
        xbc = zz[..., H * P:H * P + C]
        hist = np.zeros((Bsz, K - 1, C)) if state is None else np64(state)
        full = np.concatenate([hist, xbc], 1)
        gout = np.concatenate([np64(dx).reshape(Bsz, L, -1), np64(dB).reshape(Bsz, L, -1), np64(dC).reshape(Bsz, L, -1)], -1)
        big = np.abs(gout) * 1.2                      # |dpre| <= 1.1 |dout| (|silu'| <= 1.1)
        sw = np.stack([np.sqrt(((big * full[:, k:k + L]) ** 2).sum((0, 1))) for k in range(K)], -1)
        check_sum(dcw, ref[2], sw, dtype, f"dconv_w {tag}")
        check_sum(dcb, ref[3], np.sqrt((big ** 2).sum((0, 1))), dtype, f"dconv_b {tag}")
        check_sum(ddb, ref[4], np.sqrt((np64(ddt) ** 2).sum((0, 1))), dtype, f"ddt_bias {tag}")


@pytest.mark.parametrize("dtype,with_reset", [(torch.float32, False), (torch.float32, True), (torch.bfloat16, True)])
def test_block_backward_matches_the_oracle(dtype, with_reset):
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=3)
    Bsz, L = 2, 130
    g = torch.Generator().manual_seed(23)
    u = torch.randn(Bsz, L, 64, generator=g).to(dtype).cuda()
    dout = torch.randn(Bsz, L, 64, generator=g).to(dtype).cuda()
    reset = None
    if with_reset:
        reset = torch.zeros(Bsz, L, dtype=torch.uint8)
        reset[0, [40, 41, 100]] = 1
        reset[1, 0] = 1
    out, ctx = b.forward(u, reset=None if reset is None else reset.cuda(), save_for_backward=True)
    got = b.backward(ctx, dout)
    torch.cuda.synchronize()
    from test_gpu_block import oracle_params
    p = oracle_params(b)
    ref = blk.block_backward(np64(u), p, np64(dout), reset=None if reset is None else reset.numpy())
    # float32 runs the projections on hipBLASLt in float32 and the scan at 1e-4; bf16 rounds every tensor between the
    # stages once (about eight of them in the chain forward and back): the bars of the forward block test
    tol = 2e-3 if dtype == torch.float32 else 1.5e-1
    for key in ("du", "din_proj", "dconv_w", "dconv_b", "ddt_bias", "dA", "dD", "dnorm_w", "dout_proj"):
        o = got[key].detach().float().cpu().numpy().astype(np.float64)
        r = ref[key]
        e = np.abs(o - r).max() / max(np.sqrt(np.mean(r * r)), 1e-30)
        assert np.isfinite(o).all() and e <= tol, f"{key}: {e:.3e}"
        if dtype == torch.bfloat16:
            assert np.corrcoef(o.ravel(), r.ravel())[0, 1] > 0.999, key


def test_block_backward_is_the_directional_derivative_of_the_gpu_forward():
    """The GPU block's own forward, float32: (loss(u + h v) - loss(u - h v)) / 2h against <du, v>."""
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=4)
    g = torch.Generator().manual_seed(24)
    u = torch.randn(2, 96, 64, generator=g).cuda()
    v = torch.randn(2, 96, 64, generator=g).cuda()
    dout = torch.randn(2, 96, 64, generator=g).cuda()
    _, ctx = b.forward(u, save_for_backward=True)
    du = b.backward(ctx, dout)["du"]
    h = 1e-2
    up = (b.forward(u + h * v).double() * dout.double()).sum()
    dn = (b.forward(u - h * v).double() * dout.double()).sum()
    num = float((up - dn) / (2 * h))
    ana = float((du.double() * v.double()).sum())
    assert abs(num - ana) <= 2e-3 * max(abs(ana), 1.0), (num, ana)


@pytest.mark.parametrize("d_conv", [2, 3])
def test_block_backward_with_short_filters_at_training_size(d_conv):
    """A block with a filter shorter than four taps at 32 768 rows: the two backward stages share one scratch buffer
    sized from the filter length, and from this many rows on its conv part is the larger one, so both stages must be
    told the same length.  The size also sends the weight gradients through their slabbed path and the projections
    through the library's kernel."""
    b = Mamba2Block(d_model=128, nheads=8, headdim=16, dstate=16, ngroups=1, d_conv=d_conv, seed=5)
    Bsz, L = 8, 4096
    g = torch.Generator().manual_seed(25 + d_conv)
    u = torch.randn(Bsz, L, 128, generator=g).to(torch.bfloat16).cuda()
    dout = torch.randn(Bsz, L, 128, generator=g).to(torch.bfloat16).cuda()
    out, ctx = b.forward(u, save_for_backward=True)
    got = b.backward(ctx, dout)
    torch.cuda.synchronize()
    from test_gpu_block import oracle_params
    ref = blk.block_backward(np64(u), oracle_params(b), np64(dout))
    for key in ("du", "din_proj", "dconv_w", "dconv_b", "ddt_bias", "dA", "dD", "dnorm_w", "dout_proj"):
        o = got[key].detach().float().cpu().numpy().astype(np.float64)
        r = ref[key]
        assert o.shape == r.shape, key
        # The chain rounds to bf16 about eight times forward and back; the small block test's bar (1.5e-1 rms on the
        # worst of a few thousand elements) is a tail bound, and du here has four million elements: its worst element
        # lies further out in the same error distribution.  So: the error's own rms within 5e-2 of the reference's,
        # and its worst element within six times that (plus a share of the element for du, which is stored in bf16).
        rms = max(np.sqrt(np.mean(r * r)), 1e-30)
        err = np.abs(o - r)
        assert np.isfinite(o).all(), key
        assert np.sqrt(np.mean(err * err)) <= 5e-2 * rms, f"{key}: rms error {np.sqrt(np.mean(err * err)) / rms:.3e} rms"
        over = err - (3e-1 * rms + (2.0 ** -6 * np.abs(r) if key == "du" else 0.0))
        assert over.max() <= 0, f"{key}: over the bar by {over.max() / rms:.3e} rms"
        assert np.corrcoef(o.ravel(), r.ravel())[0, 1] > 0.999, key


@pytest.mark.parametrize("rows,e,ld,d", [(16384, 648, 704, 256), (32768, 256, 256, 64), (8192, 40, 64, 128)])
def test_weight_gradient_slabs_against_float64(rows, e, ld, d):
    """a^T b over many rows (bf16): the slabbed batched product with float32 partial sums, fed a view into wider
    rows as the block's backward does, against the float64 product of the same bf16 values.  Each output is a sum of
    `rows` products rounded once each to float32 at most: within 1e-3 of the summed terms' 2-norm."""
    from trading_bot_0_amd.block import _weight_gradient
    g = torch.Generator().manual_seed(rows + e)
    buf = torch.randn(rows, ld, generator=g).to(torch.bfloat16).cuda()
    a = buf[:, :e]
    bm = torch.randn(rows, d, generator=g).to(torch.bfloat16).cuda()
    got = _weight_gradient(a, bm)
    torch.cuda.synchronize()
    assert got.shape == (e, d) and got.dtype == torch.float32
    a64, b64 = a.double().cpu().numpy(), bm.double().cpu().numpy()
    ref = a64.T @ b64
    scale = np.sqrt((a64 * a64).sum(0))[:, None] * np.abs(b64).max()
    err = (np.abs(got.double().cpu().numpy() - ref) / scale).max()
    assert err <= 1e-3, f"{err:.3e}"
    assert torch.equal(got, _weight_gradient(a, bm)), "the same bits on a second run"
