"""daisy_decode_fwd_noalloc (the entry point that allocates nothing: its split partials live in a
buffer of the library's device image) against daisy_decode_fwd, through the C ABI, bit for bit, on
two calls in a row, the second with a smaller input; and its refusal of sizes beyond the buffer."""
import ctypes

import pytest
import torch

from daisy_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(entry, q, kn, vn, kc, vc, o, n_rows, new_idx, nsplit, workspace=None):
    lib = _lib.load()
    s2 = lambda t: _lib.strides(t, (0, 1))
    s3 = lambda t: _lib.strides(t, (0, 1, 2))
    B, H, D = q.shape
    head = (q.data_ptr(), s2(q), kn.data_ptr(), s2(kn), vn.data_ptr(), s2(vn), kc.data_ptr(), s3(kc), vc.data_ptr(), s3(vc),
            None, None, o.data_ptr(), s2(o), B, H, D, n_rows, new_idx, 1, 0.12, nsplit)
    stream = _lib.current_stream(q.device)
    if entry == "noalloc":
        return lib.daisy_decode_fwd_noalloc(*head, stream)
    ws_bytes = 0 if workspace is None else workspace.numel()
    return lib.daisy_decode_fwd(*head, _lib.ptr(workspace), ws_bytes, stream)


def _case(B, H, D, W, n_rows, new_idx, nsplit, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV).bfloat16()
    q, kn, vn = rn(B, H, D), rn(B, H, D), rn(B, H, D)
    kc, vc = rn(B, H, W, D), rn(B, H, W, D)
    lib = _lib.load()
    need = int(lib.daisy_decode_workspace_bytes(B, H, D, n_rows, nsplit))
    assert 0 < need <= _lib.DECODE_STATIC_SCRATCH_BYTES, need          # the case must really use the scratch buffer
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    kc1, vc1, kc2, vc2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
    o1 = torch.zeros(B, H, D, dtype=torch.bfloat16, device=DEV)
    o2 = torch.zeros_like(o1)
    rc = _call("workspace", q, kn, vn, kc1, vc1, o1, n_rows, new_idx, nsplit, ws)
    assert rc == 0, lib.daisy_last_error()
    assert lib.daisy_decode_noalloc_init() == 0, lib.daisy_last_error()
    torch.cuda.synchronize()
    # Free device memory as the HIP runtime reports it (hipMemGetInfo), not torch's allocator statistics: an
    # allocation made by the library itself would show here.
    free_before, _ = torch.cuda.mem_get_info(DEV)
    before = torch.cuda.memory_allocated(DEV)
    rc = _call("noalloc", q, kn, vn, kc2, vc2, o2, n_rows, new_idx, nsplit)
    assert rc == 0, lib.daisy_last_error()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(DEV)
    assert free_after >= free_before, f"free device memory fell by {free_before - free_after} bytes during the call"
    assert torch.cuda.memory_allocated(DEV) == before
    assert torch.isfinite(o2.float()).all()
    assert torch.equal(o1, o2), f"outputs differ: {(o1.float() - o2.float()).abs().max().item()}"
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2), "the appended rows differ"


def test_no_alloc_decode_equals_the_workspace_entry_point_twice_in_a_row():
    print("no-alloc decode: B2 H4 D128, 4096 live rows, 8 splits", flush=True)
    _case(B=2, H=4, D=128, W=4096, n_rows=4096, new_idx=17, nsplit=8, seed=1)
    print("no-alloc decode: smaller second call, B1 H2 D64, 700 live rows of a ring of 1024, 2 splits", flush=True)
    _case(B=1, H=2, D=64, W=1024, n_rows=700, new_idx=699, nsplit=2, seed=2)
    print("no-alloc decode: the split count chosen by the library", flush=True)
    _case(B=3, H=8, D=128, W=2048, n_rows=2048, new_idx=0, nsplit=0, seed=3)


def test_no_alloc_decode_recorded_into_a_graph():
    """The entry point under HIP graph capture (one of the callers it exists for): set up outside the capture,
    recorded once, replayed with new inputs and with eager work and synchronisations between the replays; every
    replay equals daisy_decode_fwd on the same inputs bit for bit."""
    lib = _lib.load()
    B, H, D, W, nsplit = 2, 4, 128, 2048, 4
    g = torch.Generator(device=DEV).manual_seed(9)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV).bfloat16()
    q, kn, vn = rn(B, H, D), rn(B, H, D), rn(B, H, D)
    kc, vc = rn(B, H, W, D), rn(B, H, W, D)
    o = torch.zeros(B, H, D, dtype=torch.bfloat16, device=DEV)
    assert lib.daisy_decode_noalloc_init() == 0, lib.daisy_last_error()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = _call("noalloc", q, kn, vn, kc, vc, o, W, 5, nsplit)
    assert rc == 0, lib.daisy_last_error()
    need = int(lib.daisy_decode_workspace_bytes(B, H, D, W, nsplit))
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    for it in range(4):
        print(f"no-alloc decode in a graph: replay {it}", flush=True)
        q.copy_(rn(B, H, D)); kn.copy_(rn(B, H, D)); vn.copy_(rn(B, H, D))      # eager work between the replays
        kc_ref, vc_ref = kc.clone(), vc.clone()
        o_ref = torch.zeros_like(o)
        assert _call("workspace", q, kn, vn, kc_ref, vc_ref, o_ref, W, 5, nsplit, ws) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref), f"replay {it}: outputs differ by {(o.float() - o_ref.float()).abs().max().item()}"
        assert torch.equal(kc, kc_ref) and torch.equal(vc, vc_ref), f"replay {it}: the appended rows differ"


def test_no_alloc_decode_refuses_sizes_beyond_its_buffer():
    lib = _lib.load()
    B, H, D, W, nsplit = 64, 16, 128, 512, 16          # 64*16*16*130*4 bytes = 8.5 MB of partials
    assert int(lib.daisy_decode_workspace_bytes(B, H, D, W, nsplit)) > _lib.DECODE_STATIC_SCRATCH_BYTES
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    q, kc = z(B, H, D), z(B, H, W, D)
    rc = _call("noalloc", q, q, q, kc, kc, z(B, H, D), W, 0, nsplit)
    assert rc == -3 and "built-in" in lib.daisy_last_error().decode()
