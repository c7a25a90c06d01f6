"""ssd_chunk_scan_noalloc_fwd -- the forward for callers that cannot allocate device memory -- through the C ABI,
against ssd_chunk_scan_reset_fwd with a caller-owned workspace: the same kernels on a different scratch buffer, so
y and the final states must be equal bit for bit.  Each case makes two calls in a row on the library's static
scratch array, the second with a smaller input (the array still holds the first call's intermediates), and checks
that the device's free memory does not move across the calls.

The comparison is with the workspace entry point, not with the oracle: the two run the same kernels and differ only in
the base pointer of the scratch they are handed (same layout behind it), so a bug in that layout would corrupt both
alike and is what the workspace entry point's own tests against the oracle (tests/test_gpu_scan.py) are for; what this
file can catch is what is particular to the static array: its address, its size limit, stale contents."""
from ctypes import byref, c_size_t

import pytest
import torch

from trading_bot_0_amd import ssd
from trading_bot_0_amd.synthetic import WORKLOADS, make_inputs

pytestmark = pytest.mark.gpu


def run_pair(lib, w, seqlen, with_reset, with_init):
    inp = make_inputs(w, seed=3, device="cuda", seqlen=seqlen)
    x, dt, A, Bm, Cm, D = (inp[k] for k in ("x", "dt", "A", "B", "C", "D"))
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    dims = ssd.SsdDims(Bsz, L, H, P, N, G, w.chunk)
    code = ssd.SSD_DTYPE_BF16 if x.dtype == torch.bfloat16 else ssd.SSD_DTYPE_F32
    init = torch.randn(Bsz, H, P, N, device="cuda") if with_init else None
    reset = None
    if with_reset:
        reset = torch.zeros(Bsz, L, dtype=torch.uint8, device="cuda")
        reset[0, L // 3] = 1
        reset[Bsz - 1, 0] = 1
    need = c_size_t(0)
    ssd._check(lib, lib.ssd_workspace_bytes(byref(dims), byref(need)))
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    y_ref, y_new = torch.full_like(x, float("nan")), torch.full_like(x, float("nan"))
    f_ref = torch.full((Bsz, H, P, N), float("nan"), device="cuda")
    f_new = f_ref.clone()
    stream = torch.cuda.current_stream().cuda_stream
    common = (x.data_ptr(), dt.data_ptr(), A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), D.data_ptr(), ssd._ptr(init),
              ssd._ptr(reset))
    ssd._check(lib, lib.ssd_chunk_scan_reset_fwd(byref(dims), code, *common, y_ref.data_ptr(), f_ref.data_ptr(),
                                                 ws.data_ptr(), ws.numel(), stream))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    ssd._check(lib, lib.ssd_chunk_scan_noalloc_fwd(byref(dims), code, *common, y_new.data_ptr(), f_new.data_ptr(), stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    assert not torch.isnan(y_ref.float()).any()
    assert torch.equal(y_new, y_ref), "y differs from the workspace entry point's"
    assert torch.equal(f_new, f_ref), "final states differ from the workspace entry point's"
    return need.value


def prime(lib):
    """One tiny call first: the runtime places the library's device globals (the scratch array among them) on the GPU
    when it first needs them, which is not an allocation of the call but would show in the free-memory check."""
    w = WORKLOADS["plumbing_f32"].with_batch(1)
    inp = make_inputs(w, seed=0, device="cuda", seqlen=64)
    dims = ssd.SsdDims(1, 64, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk)
    y = torch.empty_like(inp["x"])
    ssd._check(lib, lib.ssd_chunk_scan_noalloc_fwd(byref(dims), ssd.SSD_DTYPE_F32, inp["x"].data_ptr(), inp["dt"].data_ptr(),
                                                   inp["A"].data_ptr(), inp["B"].data_ptr(), inp["C"].data_ptr(), None, None,
                                                   None, y.data_ptr(), None, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()


CASES = [
    # (workload, first call (batch, seqlen), second, smaller call (batch, seqlen))
    ("policy_bf16", (32, 2048), (4, 300)),      # the one-pass kernel on segments (segment states in scratch), then staged
    ("plumbing_f32", (4, 256), (2, 100)),       # staged float32, ragged second length
    ("policy_bf16", (160, 512), (8, 512)),      # one launch of the one-pass kernel (no scratch), then staged
    ("long_lookback_bf16", (2, 1024), (1, 256)),
]


def test_noalloc_forward_takes_a_mid_size_batch_whose_staged_workspace_would_not_fit():
    """64 sequences of 4096 steps: ssd_workspace_bytes (laid out for the staged kernels) is 168 MB, but the shape runs
    on segments of the sequence and needs the segment states only (13 MB), which the static array holds."""
    lib = ssd.load_library()
    torch.cuda.set_device(0)
    prime(lib)
    w = WORKLOADS["decay_extreme"]
    assert ssd.chunk_scan_segments(w.batch, w.seqlen, w.nheads, w.headdim, w.dstate, w.ngroups, w.chunk) > 1
    need = run_pair(lib, w, w.seqlen, with_reset=True, with_init=True)
    assert need > (64 << 20)
    run_pair(lib, w.with_batch(40), 2048, with_reset=False, with_init=False)


@pytest.mark.parametrize("name,first,second", CASES)
def test_noalloc_forward_equals_the_workspace_forward_twice_in_a_row(name, first, second):
    lib = ssd.load_library()
    torch.cuda.set_device(0)
    prime(lib)
    for i, (batch, seqlen) in enumerate((first, second)):
        need = run_pair(lib, WORKLOADS[name].with_batch(batch), seqlen, with_reset=(i == 0), with_init=(i == 1))
        assert need <= (64 << 20)


def test_noalloc_forward_takes_the_full_policy_shape_and_refuses_what_does_not_fit():
    """Batch 256 at the policy shape needs 302 MB of workspace on the staged path but runs as one launch of the
    one-pass kernel, so the no-alloc entry point takes it; the same batch with heads of 16 (which only the staged
    kernels take) is refused."""
    lib = ssd.load_library()
    prime(lib)
    w = WORKLOADS["policy_bf16"]
    run_pair(lib, w, w.seqlen, with_reset=False, with_init=True)
    inp = make_inputs(w, seed=0, device="cuda")
    x16 = inp["x"][..., :16].contiguous()
    dims = ssd.SsdDims(w.batch, w.seqlen, w.nheads, 16, w.dstate, w.ngroups, w.chunk)
    y = torch.empty_like(x16)
    rc = lib.ssd_chunk_scan_noalloc_fwd(byref(dims), ssd.SSD_DTYPE_BF16, x16.data_ptr(), inp["dt"].data_ptr(), inp["A"].data_ptr(),
                                        inp["B"].data_ptr(), inp["C"].data_ptr(), None, None, None, y.data_ptr(), None, None)
    assert rc == 3 and "static scratch" in ssd.last_error(lib)


@pytest.mark.parametrize("name,batch,seqlen", [("policy_bf16", 4, 300), ("policy_bf16", 32, 2048)])
def test_noalloc_forward_captured_in_a_graph(name, batch, seqlen):
    """One staged and one segmented shape: a call outside the capture first (it places the array, asks for occupancy
    figures and raises LDS limits), then the same call captured in a graph and replayed twice with eager work and
    synchronisation between the replays; every replay must equal the workspace entry point bit for bit."""
    lib = ssd.load_library()
    torch.cuda.set_device(0)
    prime(lib)
    w = WORKLOADS[name].with_batch(batch)
    inp = make_inputs(w, seed=5, device="cuda", seqlen=seqlen)
    x, dt, A, Bm, Cm, D = (inp[k] for k in ("x", "dt", "A", "B", "C", "D"))
    Bsz, L, H, P = x.shape
    G, N = Bm.shape[2], Bm.shape[3]
    segments = ssd.chunk_scan_segments(Bsz, L, H, P, N, G, w.chunk)
    assert (segments > 1) == (batch == 32)
    dims = ssd.SsdDims(Bsz, L, H, P, N, G, w.chunk)
    reset = torch.zeros(Bsz, L, dtype=torch.uint8, device="cuda")
    reset[1, L // 2] = 1
    need = c_size_t(0)
    ssd._check(lib, lib.ssd_workspace_bytes(byref(dims), byref(need)))
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    y_ref, f_ref = torch.empty_like(x), torch.empty(Bsz, H, P, N, device="cuda")
    y_new, f_new = torch.empty_like(x), torch.empty(Bsz, H, P, N, device="cuda")

    def common(xx):
        return (xx.data_ptr(), dt.data_ptr(), A.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), D.data_ptr(), None,
                reset.data_ptr())

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # the call of this shape outside the capture
        ssd._check(lib, lib.ssd_chunk_scan_noalloc_fwd(byref(dims), ssd.SSD_DTYPE_BF16, *common(x), y_new.data_ptr(),
                                                       f_new.data_ptr(), side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ssd._check(lib, lib.ssd_chunk_scan_noalloc_fwd(byref(dims), ssd.SSD_DTYPE_BF16, *common(x), y_new.data_ptr(),
                                                       f_new.data_ptr(), torch.cuda.current_stream().cuda_stream))
    for replay in range(2):
        x.copy_(torch.randn(x.shape, device="cuda").to(x.dtype))   # eager work between the replays: new inputs
        y_new.fill_(float("nan"))
        f_new.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        ssd._check(lib, lib.ssd_chunk_scan_reset_fwd(byref(dims), ssd.SSD_DTYPE_BF16, *common(x), y_ref.data_ptr(),
                                                     f_ref.data_ptr(), ws.data_ptr(), ws.numel(),
                                                     torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert not torch.isnan(y_new.float()).any()
        assert torch.equal(y_new, y_ref) and torch.equal(f_new, f_ref), f"replay {replay}"
