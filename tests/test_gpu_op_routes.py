"""The two host routes into the ops — the compiled TORCH_LIBRARY binding and the
Python registration that calls the C ABI through ctypes — give the same results and
the same errors, and the nine registered ops pass torch's operator-registration
checks (torch.library.opcheck: schema / mutation annotations, autograd registration,
fake-tensor and AOT-dispatch behaviour), as the reference runs them on its own ops
(tests/kernels/test_layernorm.py:59-64, tests/kernels/test_fused_quant_layernorm.py:172,
wrapper tests/kernels/utils.py:1091-1103).

The dispatcher holds one registration of the namespace per process, so the route that
is not active in this process (normally the Python one: the compiled binding is loaded
when it has been built) is checked in ONE child process with
TOKENWEAVE_AMD_NO_COMPILED_BINDING=1, which runs this file's `run_opchecks()`."""
import os
import subprocess
import sys
import unittest.mock

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import tokenweave_amd as tw  # noqa: E402
from tokenweave_amd import _custom_ops as ops  # noqa: E402
from tokenweave_amd import _lib  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
OPCHECK_TEST_UTILS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic")


def _inputs(T=7, H=1024, dtype=torch.bfloat16, seed=0):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    scale = 1.0 / (2 * H)
    x = (torch.randn(T, H, generator=g, device=DEV) * scale).to(dtype)
    r = (torch.randn(T, H, generator=g, device=DEV) * scale).to(dtype)
    w = (1.0 + 0.1 * torch.randn(H, generator=g, device=DEV)).to(dtype)
    return x, r, w


def allclose_widened(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """torch.allclose for element types that have no arithmetic kernels (fp8): compared in
    float64.  opcheck's schema test compares every tensor argument before and after the call
    with torch.allclose; the reference's wrapper patches it the same way for its fp8 ops
    (tests/kernels/utils.py:1091-1103)."""
    return bool(torch.isclose(a.double(), b.double(), rtol=rtol, atol=atol, equal_nan=equal_nan).all().item())


def run_opchecks():
    """opcheck on each of the nine registered ops with sample arguments; returns the names
    checked.  Raises on the first failure."""
    T_ = torch.ops.tokenweave_amd
    eps = 1e-5
    done = []

    def check(name, args):
        print(f"[opcheck] {name}", flush=True)
        with unittest.mock.patch("torch.allclose", new=allclose_widened):
            torch.library.opcheck(getattr(T_, name), args, test_utils=OPCHECK_TEST_UTILS, raise_exception=True)
        done.append(name)

    x, r, w = _inputs()
    check("rms_norm", (torch.empty_like(x), x, w, eps))
    check("fused_add_rms_norm", (x.clone(), r.clone(), w, eps))
    check("rms_norm_inplace", (torch.empty_like(x), x.clone(), w, eps))
    check("fused_add_rms_norm_cta", (x.clone(), r.clone(), w, 4, eps))
    P = 4
    buf = tw.PartialsBuffer(P, 7, 1024, rank=1, device=DEV)
    buf.storage.normal_(0, 0.5)
    for name in ("fused_rs_ln_ag_cta", "fused_rs_ln_cta"):
        # opcheck runs the op on copies of the tensors: `input` then no longer aliases slot
        # `rank`, which the op allows (y goes to `input`, the partials are read through mcptr)
        for cap in (0, 3):
            check(name, (buf.hidden_states(7).clone(), r.clone(), w, buf.multicast_ptr, 0, 1, P, cap, eps))
    scale = torch.tensor([0.02], dtype=torch.float32, device=DEV)
    fp8 = ops.FP8_DTYPE
    check("rms_norm_static_fp8_quant", (torch.empty(x.shape, dtype=fp8, device=DEV), x, w, scale, eps))
    check("fused_add_rms_norm_static_fp8_quant",
          (torch.empty(x.shape, dtype=fp8, device=DEV), x, r.clone(), w, scale, eps))
    for qdtype in (fp8, torch.int8):
        for res in (None, r.clone()):
            check("rms_norm_dynamic_per_token_quant",
                  (torch.empty(x.shape, dtype=qdtype, device=DEV), x, w,
                   torch.empty((x.shape[0], 1), dtype=torch.float32, device=DEV), eps, None, res))
    torch.cuda.synchronize()
    return sorted(set(done))


def test_opcheck_on_the_nine_registered_ops_active_route():
    names = run_opchecks()
    assert names == sorted(ops.SCHEMAS), names


def test_opcheck_on_the_other_route_in_a_child_process():
    """The same checks with the ops registered from Python (torch.library.Library + ctypes)."""
    if not ops.COMPILED_BINDING:
        pytest.skip("the Python registration is the active route in this process (checked above)")
    env = dict(os.environ, TOKENWEAVE_AMD_NO_COMPILED_BINDING="1")
    proc = subprocess.run([sys.executable, "-u", os.path.abspath(__file__)], env=env, cwd=ROOT, timeout=300,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    print(proc.stdout[-3000:], flush=True)
    assert proc.returncode == 0, proc.stdout[-3000:]
    assert "opcheck ok: python registration" in proc.stdout


# ---------------------------------------------------------------------------
# both routes, same bits and same errors
# ---------------------------------------------------------------------------
ROUTES = [pytest.param(ops, id="active"), pytest.param(ops.via_ctypes, id="ctypes")]


def bits(t):
    return t.detach().cpu().view(torch.int16).numpy().copy()


@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_baseline_ops_both_routes(route, dtype):
    x, r, w = _inputs(33, 2048, dtype, seed=3)
    layer = tw.RMSNorm(2048, eps=1e-5, dtype=dtype).to(DEV)
    layer.weight.data.copy_(w)
    y_ref, r_ref = layer.forward_native(x, r)
    xi, ri = x.clone(), r.clone()
    route.fused_add_rms_norm(xi, ri, w, 1e-5)
    out = torch.empty_like(x)
    route.rms_norm(out, x, w, 1e-5)
    torch.cuda.synchronize()
    torch.testing.assert_close(xi, y_ref, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(ri, r_ref, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(out, layer.forward_native(x), atol=1e-2, rtol=1e-2)
    # the routes agree bit for bit
    xa, ra = x.clone(), r.clone()
    ops.fused_add_rms_norm(xa, ra, w, 1e-5)
    torch.cuda.synchronize()
    assert np.array_equal(bits(xa), bits(xi)) and np.array_equal(bits(ra), bits(ri))


@pytest.mark.parametrize("route", ROUTES)
@pytest.mark.parametrize("T", [1, 8, 48, 200, 256])
def test_fused_rs_ln_ag_cta_uncapped_both_routes(oracle, route, T):
    """MAX_CTAS = 0 and at most 256 rows: both routes send the call through the workspace
    entry point (split rows up to 48 rows at this hidden size); same bits as the capped call,
    parity with the CPU checker."""
    from helpers import assert_parity, to_bits
    from tokenweave_amd import workloads as wl
    ws, rank, H = 8, 2, 8192
    cfg = wl.NormConfig("routes", P=ws, T=T, H=H, eps=1e-5, seed=400 + T, partial_std=ws ** -0.5)
    inp = wl.make_norm_inputs(cfg, DEV)
    outs = []
    for cap in (0, max(T, 1)):
        buf = tw.PartialsBuffer(ws, T, H, rank=rank, device=DEV)
        buf.storage.copy_(inp.staging)
        res = inp.residual.clone()
        route.fused_rs_ln_ag_cta(buf.hidden_states(T), res, inp.weight, buf.multicast_ptr, 0, rank, ws, cap, cfg.eps)
        torch.cuda.synchronize()
        outs.append((to_bits(buf.hidden_states(T)), to_bits(res)))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    y_w, r_w = oracle.reduce_add_rms_norm([to_bits(p) for p in inp.partials], to_bits(inp.residual),
                                          to_bits(inp.weight), cfg.eps)
    assert_parity(outs[0][0], outs[0][1], y_w, r_w, f"route T={T}")


@pytest.mark.parametrize("route", ROUTES)
def test_error_messages_both_routes(route):
    x, r, w = _inputs(4, 1024)
    with pytest.raises(RuntimeError, match="no CPU implementation|GPU only"):
        route.fused_add_rms_norm(x.cpu(), r.cpu(), w.cpu(), 1e-5)
    with pytest.raises(NotImplementedError, match="not implemented for"):
        route.fused_add_rms_norm_cta(x.float(), r.float(), w.float(), 4, 1e-5)
    with pytest.raises(RuntimeError, match="same shape"):
        route.fused_add_rms_norm(x, r[:2], w, 1e-5)
    with pytest.raises(RuntimeError, match="row-contiguous"):
        route.rms_norm(torch.empty_like(x), x.t().contiguous().t(), w, 1e-5)
    with pytest.raises(RuntimeError, match="not inside slot 0 of a registered partials region"):
        route.fused_rs_ln_ag_cta(x, r, w, x.data_ptr(), 0, 0, 8, 0, 1e-5)
    buf = tw.PartialsBuffer(4, 4, 1024, device=DEV)
    with pytest.raises(RuntimeError, match="Invalid rank"):
        route.fused_rs_ln_cta(buf.hidden_states(4), r, w, buf.multicast_ptr, 0, 4, 4, 0, 1e-5)
    odd = torch.zeros(4 * 1032 + 8, dtype=torch.bfloat16, device=DEV)[4:4 + 4 * 1028].view(4, 1028)
    with pytest.raises(RuntimeError, match="16-byte aligned and hidden_size must be divisible by 8"):
        route.fused_add_rms_norm_cta(odd, odd.clone(), torch.ones(1028, dtype=torch.bfloat16, device=DEV), 2, 1e-5)


# ---------------------------------------------------------------------------
# decode-size calls under HIP-graph capture
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("prepared", [True, False])
def test_capture_of_the_op_itself_never_allocates(prepared):
    """torch.cuda.graph around fused_rs_ln_ag_cta(MAX_CTAS = 0) on a decode batch.  With the
    capture stream's workspace made beforehand the graph holds the split-row kernel; without
    it the op records the one-workgroup kernel instead of allocating inside the capture.
    Either way every replay equals the eager result, with eager work between replays."""
    from helpers import to_bits
    from tokenweave_amd import workloads as wl
    ws, rank, T, H = 8, 0, 8, 8192
    cfg = wl.NormConfig("capture", P=ws, T=T, H=H, eps=1e-5, seed=500, partial_std=ws ** -0.5)
    inp = wl.make_norm_inputs(cfg, DEV)
    buf = tw.PartialsBuffer(ws, T, H, rank=rank, device=DEV)
    res = inp.residual.clone()

    def reset():
        buf.storage.copy_(inp.staging)
        res.copy_(inp.residual)

    reset()
    ops.fused_rs_ln_ag_cta(buf.hidden_states(T), res, inp.weight, buf.multicast_ptr, 0, rank, ws, 0, cfg.eps)
    torch.cuda.synchronize()
    want = (to_bits(buf.hidden_states(T)), to_bits(res))

    s = torch.cuda.Stream()      # a stream no eager call has used: it has no workspace yet
    if prepared:
        ops.prepare_split_workspace(DEV, s)
    before = torch.cuda.memory_allocated()
    g = torch.cuda.CUDAGraph()
    reset()
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=s):
        ops.fused_rs_ln_ag_cta(buf.hidden_states(T), res, inp.weight, buf.multicast_ptr, 0, rank, ws, 0, cfg.eps)
    # (torch's capture itself keeps about a kilobyte of generator state; a workspace is 96 KiB)
    assert torch.cuda.memory_allocated() - before < _lib.TW_SPLIT_WORKSPACE_BYTES // 2, \
        "the captured call allocated a workspace"
    for _ in range(4):
        reset()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(to_bits(buf.hidden_states(T)), want[0]) and np.array_equal(to_bits(res), want[1])


if __name__ == "__main__":
    # child of test_opcheck_on_the_other_route_in_a_child_process
    assert torch.cuda.is_available()
    route = "compiled binding" if ops.COMPILED_BINDING else "python registration"
    names = run_opchecks()
    assert names == sorted(ops.SCHEMAS), names
    print(f"opcheck ok: {route}: {', '.join(names)}", flush=True)
