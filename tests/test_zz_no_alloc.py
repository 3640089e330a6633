"""The attention entry point that allocates nothing (cuthip_attn_decode_static: partial results in a device array
inside the library) against cuthip_attn_decode with a caller workspace, through the C ABI.  Both run the same
kernels, so the outputs must be identical bit for bit; the oracle bounds them as in test_gpu_decode_step.  Two calls
in a row share the array, the second with a smaller problem, and the array's old contents must not leak into it."""
import ctypes as C
import math

import numpy as np
import pytest

import oracle
from helpers import normwise_rel_err

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _case(lib, n_heads, n_kv, hd, seq, max_ctx, seed):
    from cut_amd import lib as L
    rng = np.random.default_rng(seed)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    K = (rng.standard_normal((max_ctx, n_kv * hd)) * 0.5).astype(np.float16)
    V = rng.standard_normal((max_ctx, n_kv * hd)).astype(np.float16)
    scale = 1 / math.sqrt(hd)
    want = oracle.attention_decode(q, K.view(np.uint16), V.view(np.uint16), seq, n_heads, n_kv, hd, scale)
    qd, Kd, Vd = dev(q), dev(K), dev(V)
    params = dev(np.array([seq - 1, seq], np.int32))
    ws_bytes = lib.cuthip_attn_decode_workspace_bytes(n_heads, hd, max_ctx)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    out_ws = torch.empty(n_heads * hd, dtype=torch.float32, device="cuda")
    out_st = torch.full((n_heads * hd,), float("nan"), dtype=torch.float32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    L.check(lib.cuthip_attn_decode(qd.data_ptr(), L.F32, Kd.data_ptr(), Vd.data_ptr(), params.data_ptr(), out_ws.data_ptr(),
                                   L.F32, n_heads, n_kv, hd, n_kv * hd, scale, max_ctx, ws.data_ptr(), ws_bytes, stream))
    L.check(lib.cuthip_attn_decode_static(qd.data_ptr(), L.F32, Kd.data_ptr(), Vd.data_ptr(), params.data_ptr(),
                                          out_st.data_ptr(), L.F32, n_heads, n_kv, hd, n_kv * hd, scale, max_ctx, stream))
    torch.cuda.synchronize()
    a, b = out_ws.cpu().numpy(), out_st.cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), "static-scratch attention differs from the workspace one"
    assert normwise_rel_err(b, want) < 2e-6   # fp32 out, as test_attention_decode


def test_static_scratch_attention_two_calls_second_smaller():
    from cut_amd import lib as L
    lib = L.load()
    L.check(lib.cuthip_init(0))
    assert lib.cuthip_attn_decode_static_max_bytes() == 4 << 20
    _case(lib, 32, 8, 128, 2048, 2048, seed=1)   # the 8B decode shape: 532,480 bytes of partials
    _case(lib, 8, 2, 64, 77, 128, seed=2)        # smaller heads, shorter cache: reuses the front of the array
    _case(lib, 6, 1, 128, 130, 256, seed=3)


def test_static_scratch_attention_rejects_oversize():
    from cut_amd import lib as L
    lib = L.load()
    L.check(lib.cuthip_init(0))
    n_heads, n_kv, hd, max_ctx = 32, 8, 128, 32768   # 17 MB of partials
    assert lib.cuthip_attn_decode_workspace_bytes(n_heads, hd, max_ctx) > lib.cuthip_attn_decode_static_max_bytes()
    t = torch.zeros(16, dtype=torch.float32, device="cuda")   # never dereferenced: the call must fail before any launch
    rc = lib.cuthip_attn_decode_static(t.data_ptr(), L.F32, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), L.F32,
                                       n_heads, n_kv, hd, n_kv * hd, 1.0, max_ctx, None)
    assert rc == -1
    assert b"built-in scratch" in lib.cuthip_last_error()
    torch.cuda.synchronize()
