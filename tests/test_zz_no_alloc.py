"""rockamdLaunchStaticWorkspace: the launch entry point that allocates nothing
(the workspace of a multi-kernel problem is an array in the library's own
device image) must produce exactly what rockamdLaunch produces with a
caller-allocated workspace.  Two problems in a row, the second smaller, so
that stale contents of the shared array would show."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _kernels(rock, opts):
    first = rock.RockKernel(opts)
    return [first] + [rock.RockKernel("%s --kernel_id %d" % (opts, i)) for i in range(1, first.kernel_count)]


def _launch_static(rock, kern, tensors):
    lib = rock.load_library()
    arr = (C.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])
    stream = torch.cuda.current_stream().cuda_stream
    return lib.rockamdLaunchStaticWorkspace(kern._h, arr, len(tensors), stream)


def _split_gemm(rock, gpu, M, N, K, seed):
    """f16 GEMM with few output tiles and a long K: K-split partial sums in a
    workspace, then the reduction kernel."""
    g = torch.Generator(device=gpu)
    g.manual_seed(seed)
    a = torch.randn((M, K), generator=g, device=gpu).half()
    b = torch.randn((K, N), generator=g, device=gpu).half()
    opts = "-operation gemm -arch gfx950 -t f16 -g 1 -m %d -n %d -k %d" % (M, N, K)
    kernels = _kernels(rock, opts)
    assert len(kernels) == 2 and kernels[0].workspace_bytes > 0
    # existing entry point, caller-allocated workspace
    ws = torch.empty(kernels[0].workspace_bytes, dtype=torch.uint8, device=gpu)
    want = torch.full((M, N), 7.0, dtype=torch.float16, device=gpu)
    for k in kernels:
        k.launch(a, b, want, None, ws)
    # the entry point under test: the same pointer list without the workspace
    got = torch.full((M, N), -7.0, dtype=torch.float16, device=gpu)
    for k in kernels:
        assert _launch_static(rock, k, (a, b, got, None)) == 0, rock.api.last_error()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    return kernels[0].workspace_bytes


def test_static_workspace_matches_caller_workspace_twice(rock, gpu):
    big = _split_gemm(rock, gpu, 128, 1280, 5120, 11)
    small = _split_gemm(rock, gpu, 64, 256, 4096, 12)   # second call, smaller problem, same shared array
    assert small < big


def test_static_workspace_conv_relayout_plan(rock, gpu):
    """A second family of multi-kernel problems: NCHW convolution = layout
    conversions into the workspace, then the contraction."""
    n, c, k, hw = 4, 32, 64, 14
    g = torch.Generator(device=gpu)
    g.manual_seed(13)
    fil = torch.randint(-2, 3, (k * c * 9,), generator=g, device=gpu).half()
    inp = torch.randint(-2, 3, (n * c * hw * hw,), generator=g, device=gpu).half()
    opts = ("--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout gkcyx "
            "--in_layout ngchw --out_layout ngkhw --batchsize %d --groupsize 1 --in_channels %d --out_channels %d "
            "--in_h %d --in_w %d --fil_h 3 --fil_w 3 --padding_h 1 --padding_w 1" % (n, c, k, hw, hw))
    kernels = _kernels(rock, opts)
    assert len(kernels) > 1 and kernels[0].workspace_bytes > 0
    ws = torch.empty(kernels[0].workspace_bytes, dtype=torch.uint8, device=gpu)
    want = torch.zeros(n * k * hw * hw, dtype=torch.float16, device=gpu)
    got = torch.ones_like(want)
    for kern in kernels:
        kern.launch(fil, inp, want, None, ws)
    for kern in kernels:
        assert _launch_static(rock, kern, (fil, inp, got, None)) == 0, rock.api.last_error()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_static_workspace_calls_allocate_no_device_memory(rock, gpu):
    """After a first pass (modules loaded, the array's address looked up), a second sequence of calls through the
    entry point leaves the device's free memory as it was: hipMemGetInfo before and after, with the tensors
    allocated beforehand."""
    g = torch.Generator(device=gpu)
    g.manual_seed(14)
    a = torch.randn((128, 5120), generator=g, device=gpu).half()
    b = torch.randn((5120, 1280), generator=g, device=gpu).half()
    got = torch.empty((128, 1280), dtype=torch.float16, device=gpu)
    kernels = _kernels(rock, "-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 1280 -k 5120")
    assert len(kernels) == 2
    for k in kernels:                                   # warm-up
        assert _launch_static(rock, k, (a, b, got, None)) == 0, rock.api.last_error()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(gpu)       # hipMemGetInfo
    for _ in range(3):
        for k in kernels:
            assert _launch_static(rock, k, (a, b, got, None)) == 0, rock.api.last_error()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(gpu)
    assert free_after == free_before
    assert torch.allclose(got.float(), a.float() @ b.float(), rtol=2e-2, atol=0.5)


def test_static_workspace_single_kernel_and_limits(rock, gpu):
    # a problem without a workspace: same list as rockamdLaunch, same result
    a = torch.randint(-128, 128, (256, 512), device=gpu, dtype=torch.int8)
    b = torch.randint(-128, 128, (128, 512), device=gpu, dtype=torch.int8)
    k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -g 1 -m 256 -n 128 -k 512 -transB true")
    want = torch.zeros((256, 128), dtype=torch.int32, device=gpu)
    got = torch.ones_like(want)
    k.launch(a, b, want, None)
    assert _launch_static(rock, k, (a, b, got, None)) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # wrong pointer count
    assert _launch_static(rock, k, (a, b, got)) != 0
    # a workspace beyond the built-in array is refused before anything is launched: the channels-last copies of
    # an NCHW convolution over 256 images of 256 x 56 x 56 (0.4 GB each way)
    big = rock.RockKernel("--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 "
                          "--fil_layout gkcyx --in_layout ngchw --out_layout ngkhw --batchsize 256 --groupsize 1 "
                          "--in_channels 256 --out_channels 256 --in_h 56 --in_w 56 --fil_h 3 --fil_w 3 "
                          "--padding_h 1 --padding_w 1")
    assert big.workspace_bytes > (64 << 20)
    x = torch.zeros(4096, dtype=torch.float16, device=gpu)   # never touched: the call is refused first
    o = torch.full_like(x, 3.0)
    rc = _launch_static(rock, big, (x, x, o, None))
    assert rc != 0 and "workspace" in rock.api.last_error()
    torch.cuda.synchronize()
    assert float(o.min()) == 3.0


def test_static_workspace_takes_chunked_attention(rock, gpu):
    """f32 attention whose scores (8 x 2048 x 2048 x 4 bytes = 128 MiB) exceed the array: the three-kernel form
    works them off in chunks of 32 MiB, so the entry point accepts the problem; results as with rockamdLaunch."""
    G, s, d = 8, 2048, 64
    g = torch.Generator(device=gpu)
    g.manual_seed(15)
    q = torch.randn((G, s, d), generator=g, device=gpu)
    k = torch.randn((G, s, d), generator=g, device=gpu)
    v = torch.randn((G, s, d), generator=g, device=gpu)
    kernels = _kernels(rock, "-operation attention -arch gfx950 -t f32 -g %d -seq_len_q %d -seq_len_k %d "
                             "-head_dim_qk %d -head_dim_v %d -transK true -scale 0.125" % (G, s, s, d, d))
    assert len(kernels) == 12 and kernels[0].workspace_bytes == (32 << 20)
    ws = torch.empty(kernels[0].workspace_bytes, dtype=torch.uint8, device=gpu)
    want = torch.zeros((G, s, d), device=gpu)
    got = torch.ones_like(want)
    for kern in kernels:
        kern.launch(q, k, v, None, want, ws)
    for kern in kernels:
        assert _launch_static(rock, kern, (q, k, v, None, got)) == 0, rock.api.last_error()
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    ref = torch.softmax((q @ k.transpose(1, 2)) * 0.125, dim=-1) @ v
    assert float((got - ref).abs().max()) < 1e-4
