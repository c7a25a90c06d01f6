"""The Mamba-2 block stages around the scan through the C ABI (pre: conv + SiLU + softplus; post: gated
RMSNorm) against the numpy oracle, and the assembled block (torch GEMMs + library kernels) against the
oracle's block, batched and streamed."""
import numpy as np
import pytest
import torch

from oracle import mamba2_block_oracle as blk
from trading_bot_0_amd import Mamba2Block, SsdError, block_post, block_post_proj, block_pre, block_proj

from _util import np64, rel_err

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def params(H, P, N, G, K, seed=0):
    g = torch.Generator().manual_seed(seed)
    C = H * P + 2 * G * N
    return dict(conv_w=torch.randn(C, K, generator=g).cuda() / 2, conv_b=torch.randn(C, generator=g).cuda() / 4,
                dt_bias=torch.randn(H, generator=g).cuda(), norm_w=torch.randn(H * P, generator=g).cuda())


def close(out, ref, dtype, what):
    """float32: max|err| / rms <= 2e-5.  bf16: these stages are elementwise and store bf16, so every element
    must be within two bf16 ulps (2^-7 relative) of the float64 result, plus a floor of 1e-3 rms for values
    that cancel to nearly zero."""
    o = out.detach().float().cpu().numpy().astype(np.float64).reshape(ref.shape)
    assert np.isfinite(o).all(), what
    if dtype == torch.float32:
        e = rel_err(out, ref)
        assert e <= TOL[dtype], f"{what}: {e:.3e}"
        return e
    rms = np.sqrt(np.mean(ref * ref))
    bad = np.abs(o - ref) > 2.0 ** -7 * np.abs(ref) + 1e-3 * rms
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off by more than two bf16 ulps"
    return 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1, 4), (3, 7, 8, 16, 16, 2, 3), (1, 130, 16, 64, 128, 2, 2),
                                   (4, 1, 8, 32, 64, 1, 4), (2, 2, 8, 32, 32, 4, 4)])
def test_pre_scan_stage(shape, dtype):
    Bsz, L, H, P, N, G, K = shape
    p = params(H, P, N, G, K)
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(1)
    z = torch.randn(Bsz, L, E, generator=g).to(dtype).cuda()
    st = (torch.randn(Bsz, K - 1, H * P + 2 * G * N, generator=g)).to(dtype).cuda()
    for state in (None, st):
        got = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=state, return_conv_state=True)
        ref = blk.block_pre(np64(z), np64(p["conv_w"]), np64(p["conv_b"]), np64(p["dt_bias"]), H, P, N, G,
                            None if state is None else np64(state))
        for name, a, b in zip(("x", "B", "C", "dt"), got[:4], ref[:4]):
            close(a, b, dtype, f"pre {name}")
        assert torch.equal(got[4].float().cpu(), torch.from_numpy(ref[4]).float()), "conv state is a copy of inputs"
        # without asking for the state the outputs are the same
        again = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=state)
        assert all(torch.equal(a, b) for a, b in zip(again, got[:4]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1), (3, 7, 8, 16, 16, 2), (1, 33, 16, 64, 128, 2), (2, 5, 32, 64, 16, 1),
                                   (2, 9, 8, 24, 16, 1), (1, 21, 24, 24, 16, 1), (3, 6, 40, 40, 16, 1)])  # rows the lanes do not cover exactly
def test_post_scan_stage(shape, dtype):
    Bsz, L, H, P, N, G = shape
    p = params(H, P, N, G, 4)
    g = torch.Generator().manual_seed(2)
    z = torch.randn(Bsz, L, 2 * H * P + 2 * G * N + H, generator=g).to(dtype).cuda()
    y = (torch.randn(Bsz, L, H, P, generator=g) * 3).to(dtype).cuda()
    ref = blk.block_post(np64(y), np64(z), np64(p["norm_w"]), 1e-5)
    close(block_post(y, z, p["norm_w"], H, P, N, G), ref, dtype, "post")
    if dtype == torch.bfloat16:      # the scan's float32 y as input
        y32 = y.float() + 1e-3
        close(block_post(y32, z, p["norm_w"], H, P, N, G), blk.block_post(np64(y32), np64(z), np64(p["norm_w"]), 1e-5),
              dtype, "post from float32 y")


def oracle_params(b):
    return dict(in_proj=np64(b.in_proj), conv_w=np64(b.conv_w), conv_b=np64(b.conv_b), dt_bias=np64(b.dt_bias),
                A=np64(b.A), D=np64(b.D), norm_w=np64(b.norm_w), out_proj=np64(b.out_proj), H=b.H, P=b.P, N=b.N, G=b.G,
                eps=b.eps)


@pytest.mark.parametrize("rows,k,n", [(300, 256, 648), (256, 128, 32), (1, 128, 264), (4099, 256, 256), (2, 256, 8),
                                      (2049, 256, 648), (70000, 128, 168)])
def test_projection_against_float64(rows, k, n):
    """out = u . w^T in bf16 with float32 accumulation: every element within one bf16 rounding of the float64
    product of the same bf16 inputs (plus a floor for sums that cancel); ragged row counts, column blocks and
    chunks."""
    g = torch.Generator().manual_seed(rows + n)
    u = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    out = block_proj(u.cuda(), w.cuda())
    torch.cuda.synchronize()
    assert out.shape == (rows, n) and out.dtype == torch.bfloat16
    ref = u.double().numpy() @ w.double().numpy().T
    o = out.float().cpu().numpy().astype(np.float64)
    rms = np.sqrt(np.mean(ref * ref))
    bad = np.abs(o - ref) > 2.0 ** -8 * np.abs(ref) + 1e-4 * rms
    assert np.isfinite(o).all() and not bad.any(), f"{int(bad.sum())} elements off"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1, 4), (3, 7, 8, 16, 16, 2, 3), (4, 1, 8, 32, 64, 1, 4)])
def test_stages_take_padded_rows(shape, dtype):
    """zxbcdt as the first E columns of a buffer with longer rows (what the in-projection writes when asked for rows
    of whole 128-byte lines): pre and post give the dense tensor's results bit for bit, whatever the padding holds."""
    Bsz, L, H, P, N, G, K = shape
    p = params(H, P, N, G, K)
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(5)
    z = torch.randn(Bsz, L, E, generator=g).to(dtype).cuda()
    buf = torch.full((Bsz, L, (E + 63) // 64 * 64 + 64), float("nan"), dtype=dtype, device="cuda")
    buf[..., :E] = z
    zp = buf[..., :E]
    assert not zp.is_contiguous() or L * Bsz == 1
    st = (torch.randn(Bsz, K - 1, H * P + 2 * G * N, generator=g)).to(dtype).cuda()
    dense = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=st, return_conv_state=True)
    padded = block_pre(zp, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=st, return_conv_state=True)
    assert all(torch.equal(a, b) for a, b in zip(dense, padded))
    y = (torch.randn(Bsz, L, H, P, generator=g) * 3).to(dtype).cuda()
    assert torch.equal(block_post(y, z, p["norm_w"], H, P, N, G), block_post(y, zp, p["norm_w"], H, P, N, G))
    with pytest.raises(ValueError):       # a view that does not start on a 16-byte piece
        block_pre(buf[:, :, 1:E + 1], p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)
    with pytest.raises(ValueError):       # elements of a row not adjacent
        block_pre(buf[:, :, :2 * E:2], p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)


@pytest.mark.parametrize("shape", [(2, 50, 8, 32, 64, 1, 256), (3, 700, 8, 32, 64, 1, 256), (1, 2049, 8, 16, 16, 1, 128),
                                   (5, 33, 16, 16, 16, 2, 72), (1, 1, 8, 32, 64, 1, 8), (2, 4100, 8, 32, 128, 1, 200)])
@pytest.mark.parametrize("padded", [False, True])
def test_post_scan_with_out_projection_in_one_kernel(shape, padded):
    """rmsnorm(y silu(z)) norm_w . w^T as one kernel against the float64 value of the same bf16 inputs.  The kernel
    rounds the gated row and the weights times norm_w to bf16 once each and the sum once more on the way out, so
    every element lies within 2^-8 of the sum of its terms' magnitudes plus one bf16 rounding of itself -- a bound
    on rounding alone; a misplaced row, channel or factor is off by the terms' 2-norm, an order of magnitude more.
    Ragged row counts (rows past the last tile), column counts off the chunks of 32, rows of whole lines."""
    Bsz, L, H, P, N, G, dm = shape
    p = params(H, P, N, G, 4)
    DI, E = H * P, 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(L + dm)
    z = torch.randn(Bsz, L, E, generator=g).to(torch.bfloat16).cuda()
    if padded:
        buf = torch.full((Bsz, L, (E + 63) // 64 * 64), float("nan"), dtype=torch.bfloat16, device="cuda")
        buf[..., :E] = z
        z = buf[..., :E]
    y = (torch.randn(Bsz, L, H, P, generator=g) * 3).to(torch.bfloat16).cuda()
    w = (torch.randn(dm, DI, generator=g) / DI ** 0.5).to(torch.bfloat16).cuda()
    out = block_post_proj(y, z, p["norm_w"], w, H, P, N, G)
    torch.cuda.synchronize()
    assert out.shape == (Bsz, L, dm) and out.dtype == torch.bfloat16
    yn = blk.block_post(np64(y), np64(z), np64(p["norm_w"]), 1e-5).reshape(Bsz * L, DI)
    w64 = np64(w)
    ref = yn @ w64.T
    mag = np.abs(yn) @ np.abs(w64).T
    o = np64(out).reshape(Bsz * L, dm)
    over = np.abs(o - ref) - (1.05 * 2.0 ** -8 * mag + 2.0 ** -8 * np.abs(ref) + 1e-30)
    assert np.isfinite(o).all() and over.max() <= 0, f"over the rounding bound by {over.max():.3e}"
    # and next to the two stages run one after the other (their bf16 roundings fall elsewhere, within the same bound)
    two = np64(block_proj(block_post(y, z, p["norm_w"], H, P, N, G), w)).reshape(Bsz * L, dm)
    assert (np.abs(o - two) <= 2 * (1.05 * 2.0 ** -8 * mag + 2.0 ** -8 * np.abs(ref)) + 1e-30).all()


@pytest.mark.parametrize("rows,k,n", [(300, 256, 648), (4099, 256, 256), (2049, 128, 168), (33, 256, 8), (5000, 256, 768)])
def test_projection_into_padded_rows(rows, k, n):
    """pad_rows: the same numbers as the dense call, bit for bit, in rows a multiple of 64 elements apart; columns
    past out_features are not written."""
    g = torch.Generator().manual_seed(rows + n)
    u = torch.randn(rows, k, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(n, k, generator=g) / k ** 0.5).to(torch.bfloat16).cuda()
    dense = block_proj(u, w)
    padded = block_proj(u, w, pad_rows=True)
    assert padded.shape == (rows, n) and padded.stride(0) == (n + 63) // 64 * 64 and padded.stride(1) == 1
    assert torch.equal(dense, padded)
    # through the C ABI into a poisoned buffer: the padding stays as it was
    from ctypes import c_void_p
    from trading_bot_0_amd import ssd
    from trading_bot_0_amd.block import _lib
    ld = (n + 63) // 64 * 64 + 64
    buf = torch.full((rows, ld), -7.0, dtype=torch.bfloat16, device="cuda")
    lib = _lib()
    ssd._check(lib, lib.ssd_block_proj_fwd(rows, k, n, ld, ssd.SSD_DTYPE_BF16, u.data_ptr(), w.data_ptr(), buf.data_ptr(),
                                           ssd._stream_ptr(u)))
    torch.cuda.synchronize()
    assert torch.equal(buf[:, :n], dense) and bool((buf[:, n:] == -7.0).all())
    for bad_ld in ((n - 8, n + 4) if n > 8 else (n + 4, n + 9)):   # (0 would mean dense)
        with pytest.raises(SsdError):
            ssd._check(lib, lib.ssd_block_proj_fwd(rows, k, n, bad_ld, ssd.SSD_DTYPE_BF16, u.data_ptr(), w.data_ptr(),
                                                   buf.data_ptr(), ssd._stream_ptr(u)))


def test_projection_keeps_leading_dimensions_and_refuses_other_shapes():
    u = torch.randn(3, 50, 256).to(torch.bfloat16).cuda()
    w = torch.randn(40, 256).to(torch.bfloat16).cuda()
    out = block_proj(u, w)
    assert out.shape == (3, 50, 40)
    ref = u.double().cpu().numpy().reshape(150, 256) @ w.double().cpu().numpy().T
    assert np.abs(out.float().cpu().numpy().reshape(150, 40) - ref).max() <= 2.0 ** -7 * np.abs(ref).max()
    with pytest.raises(SsdError):
        block_proj(torch.randn(8, 96).to(torch.bfloat16).cuda(), torch.randn(8, 96).to(torch.bfloat16).cuda())
    with pytest.raises(SsdError):
        block_proj(u, torch.randn(42, 256).to(torch.bfloat16).cuda())
    with pytest.raises(ValueError):
        block_proj(u.float(), w.float())


def test_block_forward_float32_matches_the_oracle_block():
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=3)
    u = torch.randn(2, 200, 64, generator=torch.Generator().manual_seed(4)).cuda()
    out = b.forward(u)
    ref, _, _ = blk.block_forward(np64(u), oracle_params(b))
    assert rel_err(out, ref) <= 1e-3          # float32 GEMMs (hipBLASLt) on top of the 1e-4 scan


def test_block_forward_bf16_is_close_to_the_oracle_block():
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=3)
    u = torch.randn(2, 200, 64, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).cuda()
    out = b.forward(u)
    ref, _, _ = blk.block_forward(np64(u), oracle_params(b))
    # every bf16 tensor between the stages (projection output, x, B, C, dt, y, normed y) is rounded once: 2^-9
    # each, about five of them in a chain
    assert out.dtype == torch.bfloat16 and rel_err(out, ref) <= 1e-1
    corr = np.corrcoef(out.float().cpu().numpy().ravel(), ref.ravel())[0, 1]
    assert corr > 0.9995


def test_block_streams_prefix_then_steps_equals_the_window():
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=5)
    u = torch.randn(3, 96, 64, generator=torch.Generator().manual_seed(6)).cuda()
    full = b.forward(u)
    st = b.new_state(3, dtype=torch.float32)
    outs = [b.forward(u[:, :70].contiguous(), state=st)]
    for t in range(70, 96):
        outs.append(b.step(u[:, t].contiguous(), st).unsqueeze(1))
    got = torch.cat(outs, 1)
    torch.cuda.synchronize()
    assert rel_err(got, np64(full)) <= 1e-3
    ref, conv, ssm = blk.block_forward(np64(u), oracle_params(b))
    assert rel_err(st.ssm.state, ssm) <= 1e-3 and rel_err(st.conv, conv) <= 1e-6
    # a restarted stream forgets: zero both states of row 1 and compare with a fresh stream on the same input
    st.reset_rows(torch.tensor([1], device="cuda"))
    fresh = b.new_state(3, dtype=torch.float32)
    o1 = b.step(u[:, 0].contiguous(), st)
    o2 = b.step(u[:, 0].contiguous(), fresh)
    assert torch.equal(o1[1], o2[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 50, 8, 32, 64, 1, 4), (2, 19, 8, 16, 16, 2, 3), (2, 33, 8, 32, 32, 1, 2), (3, 2, 8, 32, 64, 1, 4)])
def test_pre_scan_stage_with_restarts(shape, dtype):
    """Episode boundaries inside the window cut the conv's history: against the oracle (pinned by running the
    episodes as separate windows), with restarts on both sides of the kernel's runs of 16 timesteps, back to back,
    at the first and at the last timestep."""
    Bsz, L, H, P, N, G, K = shape
    p = params(H, P, N, G, K)
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(11)
    z = torch.randn(Bsz, L, E, generator=g).to(dtype).cuda()
    st = (torch.randn(Bsz, K - 1, H * P + 2 * G * N, generator=g)).to(dtype).cuda()
    reset = torch.zeros(Bsz, L, dtype=torch.uint8)
    for t in (0, 5, 6, 15, 16, 17, 31, 33, L - 1):
        if 0 <= t < L:
            reset[t % Bsz, t] = 1
    reset[0, L - 1] = 1
    for state in (None, st):
        got = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=state, return_conv_state=True,
                        reset=reset.cuda())
        ref = blk.block_pre(np64(z), np64(p["conv_w"]), np64(p["conv_b"]), np64(p["dt_bias"]), H, P, N, G,
                            None if state is None else np64(state), reset.numpy())
        for name, a, b in zip(("x", "B", "C", "dt"), got[:4], ref[:4]):
            close(a, b, dtype, f"pre {name} with restarts")
        assert torch.equal(got[4].float().cpu(), torch.from_numpy(ref[4]).float()), "conv state after restarts"
    # an all-zero mask is no mask
    a = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=st, return_conv_state=True)
    b_ = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=st, return_conv_state=True,
                   reset=torch.zeros(Bsz, L, dtype=torch.bool).cuda())
    assert all(torch.equal(u, v) for u, v in zip(a, b_))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [2, 3, 4])
def test_conv_state_updated_in_place_for_one_timestep(K, dtype):
    """seqlen 1 with conv_state_in == conv_state_out (what a streaming step does): the new state is the old one
    shifted by one row plus the new input row, as with separate buffers, for every filter width."""
    Bsz, H, P, N, G = 5, 8, 32, 64, 1
    p = params(H, P, N, G, K)
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(12 + K)
    st0 = torch.randn(Bsz, K - 1, H * P + 2 * G * N, generator=g).to(dtype).cuda()
    separate, inplace = st0.clone(), st0.clone()
    for step in range(K + 1):
        z = torch.randn(Bsz, 1, E, generator=g).to(dtype).cuda()
        out_a = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=separate, return_conv_state=True)
        out_b = block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G, conv_state=inplace, conv_state_out=inplace)
        torch.cuda.synchronize()
        assert out_b[4] is inplace
        assert all(torch.equal(u, v) for u, v in zip(out_a, out_b)), f"step {step}"
        ref_state = torch.cat([separate[:, 1:], z[:, :, H * P:H * P + separate.shape[2]]], 1)
        assert torch.equal(out_a[4], ref_state)
        separate = out_a[4]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_window_with_restarts_equals_the_stream_that_was_reset(dtype):
    """A replayed window with episode boundaries gives what the rollout produced: stepping the block bar by bar and
    zeroing a stream's conv and SSM state (reset_rows) before the bars the mask marks."""
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, ngroups=1, seed=7)
    Bsz, L = 3, 40
    u = torch.randn(Bsz, L, 64, generator=torch.Generator().manual_seed(8)).to(dtype).cuda()
    reset = torch.zeros(Bsz, L, dtype=torch.bool)
    reset[0, [3, 4, 20]] = True
    reset[1, 0] = True
    reset[2, [17, L - 1]] = True
    window = b.forward(u, reset=reset.cuda())
    st = b.new_state(Bsz, dtype=dtype)
    outs = []
    for t in range(L):
        rows = torch.nonzero(reset[:, t]).flatten().cuda()
        if rows.numel():
            st.reset_rows(rows)
        outs.append(b.step(u[:, t].contiguous(), st).unsqueeze(1))
    stepped = torch.cat(outs, 1)
    torch.cuda.synchronize()
    ref, _, _ = blk.block_forward(np64(u), oracle_params(b), reset=reset.numpy())
    if dtype == torch.float32:
        assert rel_err(window, ref) <= 1e-3 and rel_err(stepped, ref) <= 1e-3
        assert rel_err(window, np64(stepped)) <= 1e-3
    else:
        assert rel_err(window, ref) <= 1e-1 and rel_err(stepped, ref) <= 1e-1
        # without the cut the three bars after each restart would see the previous episode: far outside rounding
        leaky = b.forward(u)
        assert rel_err(window, np64(stepped)) < 0.25 * rel_err(leaky, np64(stepped))


def test_block_stage_errors():
    p = params(8, 32, 64, 1, 4)
    z = torch.randn(2, 4, 2 * 256 + 128 + 8).cuda()
    with pytest.raises(ValueError, match="channels"):
        block_pre(z[:, :, :-8].contiguous(), p["conv_w"], p["conv_b"], p["dt_bias"], 8, 32, 64, 1)
    with pytest.raises(SsdError) as ei:        # width-5 conv is not built
        block_pre(z, torch.randn(256 + 128, 5).cuda(), p["conv_b"], p["dt_bias"], 8, 32, 64, 1)
    assert ei.value.code == 2
    with pytest.raises(ValueError, match="conv_state"):
        block_pre(z, p["conv_w"], p["conv_b"], p["dt_bias"], 8, 32, 64, 1, conv_state=torch.zeros(2, 2, 384).cuda())


def test_block_stages_inside_a_captured_graph():
    """The library's three block kernels (projection into padded rows, pre, post) captured in one graph: replays,
    with the input changed in place and eager work in between, equal the eager calls bit for bit."""
    H, P, N, G, K = 8, 32, 64, 1, 4
    p = params(H, P, N, G, K)
    E = 2 * H * P + 2 * G * N + H
    g = torch.Generator().manual_seed(9)
    u = torch.randn(4, 300, 256, generator=g).to(torch.bfloat16).cuda()
    w_in = (torch.randn(E, 256, generator=g) / 16).to(torch.bfloat16).cuda()
    y = torch.randn(4, 300, H, P, generator=g).to(torch.bfloat16).cuda()

    def chain():
        zx = block_proj(u, w_in, pad_rows=True)
        outs = block_pre(zx, p["conv_w"], p["conv_b"], p["dt_bias"], H, P, N, G)
        return outs + (block_post(y, zx, p["norm_w"], H, P, N, G),)

    chain()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = chain()
    u_keep = u.clone()
    for i in range(4):
        for t in captured:
            t.fill_(float("nan"))
        u.copy_(u_keep * 0.5 if i % 2 else u_keep)
        graph.replay()
        torch.cuda.synchronize()
        eager = chain()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(captured, eager)), f"replay {i}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cfg", [(256, 8, 32, 64, 1, 4, 4), (128, 8, 16, 16, 2, 3, 3), (256, 16, 16, 128, 2, 2, 5),
                                 (128, 8, 32, 32, 1, 4, 1), (256, 8, 16, 32, 1, 4, 2)])
def test_block_step_as_one_launch(cfg, dtype):
    """The whole step as one kernel (ssd_block_step_fwd), three steps in a row from random states, against the float64
    oracle block run one timestep at a time from the same states, and against the stage kernels' step: outputs and
    both states.  float32: 1e-3 of the rms (the bar of the streamed block test); bf16: the block test's 1e-1 for the
    output (about five bf16 roundings in the chain) and for the SSM state (its increment dt x B is a product of three
    rounded factors, and the largest elements of it are many rms of the state); next to the stage kernels, which round
    at the same points, 1e-2."""
    d_model, H, P, N, G, K, Bsz = cfg
    b = Mamba2Block(d_model=d_model, nheads=H, headdim=P, dstate=N, ngroups=G, d_conv=K, seed=7)
    p = oracle_params(b)
    g = torch.Generator().manual_seed(31)
    C = H * P + 2 * G * N
    conv0 = torch.randn(Bsz, K - 1, C, generator=g).to(dtype).cuda()
    ssm0 = torch.randn(Bsz, H, P, N, generator=g).cuda()
    us = torch.randn(3, Bsz, d_model, generator=g).to(dtype).cuda()
    st_f, st_s = b.new_state(Bsz, dtype=dtype), b.new_state(Bsz, dtype=dtype)
    for st in (st_f, st_s):
        st.conv.copy_(conv0)
        st.ssm.state.copy_(ssm0)
    conv_ref, ssm_ref = np64(conv0), np64(ssm0)
    tol_out, tol_state = (1e-3, 1e-3) if dtype == torch.float32 else (1e-1, 1e-1)
    for i in range(3):
        out_f = b.step(us[i], st_f, fused=True)
        out_s = b.step(us[i], st_s, fused=False)
        torch.cuda.synchronize()
        ref, conv_ref, ssm_ref = blk.block_forward(np64(us[i]).reshape(Bsz, 1, d_model), p, conv_state=conv_ref, ssm_state=ssm_ref)
        assert out_f.shape == (Bsz, d_model) and out_f.dtype == dtype
        assert rel_err(out_f, ref[:, 0]) <= tol_out, f"step {i}: output {rel_err(out_f, ref[:, 0]):.3e}"
        assert rel_err(st_f.ssm.state, ssm_ref) <= tol_state, f"step {i}: SSM state"
        assert rel_err(st_f.conv, conv_ref) <= (1e-5 if dtype == torch.float32 else 2.0 ** -7 * 6), f"step {i}: conv state"
        # beside the stage kernels' step (same rounding points, other summation orders)
        assert rel_err(out_f, np64(out_s)) <= (1e-4 if dtype == torch.float32 else 5e-2), f"step {i}: fused vs stages"
        assert rel_err(st_f.ssm.state, np64(st_s.ssm.state)) <= (1e-5 if dtype == torch.float32 else 1e-2)
        # the oracle continues from its own states; the conv state it returns is the raw in-projection rows, which
        # the GPU holds rounded to the activation type: continue the oracle from the GPU's rows so that the three steps
        # test three steps, not the drift of a rounding
        conv_ref = np64(st_f.conv)


def test_block_step_as_one_launch_refuses_what_it_does_not_take():
    b = Mamba2Block(d_model=64, nheads=8, headdim=32, dstate=64, seed=1)
    st = b.new_state(2, dtype=torch.float32)
    with pytest.raises(SsdError):
        b.step(torch.randn(2, 64).cuda(), st, fused=True)
    out = b.step(torch.randn(2, 64).cuda(), st)     # the default picks the stage kernels for this width
    assert out.shape == (2, 64)


def test_graphed_step_equals_the_eager_step_on_every_replay():
    """The block's step captured in a graph (no memset nodes: every kernel writes what it later reads) and replayed
    with the program's own eager work between the replays; outputs and both states equal the eager step's bit for bit."""
    blk = Mamba2Block(d_model=256, nheads=8, headdim=32, dstate=64, seed=3)
    g = torch.Generator().manual_seed(5)
    prefix = torch.randn(4, 40, 256, generator=g).to(torch.bfloat16).cuda()
    bars = torch.randn(6, 4, 256, generator=g).to(torch.bfloat16).cuda()
    st_e, st_g = blk.new_state(4), blk.new_state(4)
    blk.forward(prefix, state=st_e)
    blk.forward(prefix, state=st_g)
    conv0, ssm0 = st_g.conv.clone(), st_g.ssm.state.clone()
    step = blk.graphed_step(st_g)
    assert torch.equal(st_g.conv, conv0) and torch.equal(st_g.ssm.state, ssm0), "building the graph moved the state"
    for i in range(bars.shape[0]):
        out_e = blk.step(bars[i], st_e)
        torch.cuda.synchronize()
        out_g = step(bars[i]).clone()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"replay {i}: output"
        assert torch.equal(st_g.conv, st_e.conv) and torch.equal(st_g.ssm.state, st_e.ssm.state), f"replay {i}: state"
        _ = (prefix.float() * 2).sum().item()      # eager work and a synchronisation between the replays
