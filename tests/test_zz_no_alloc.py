"""GPU test of qvb8_moe_experts_static: the MoE expert stack with the workspace inside the library (a call that
allocates nothing) against qvb8_moe_experts with a caller workspace, through the C ABI, bit for bit -- two calls in a row,
the second with a smaller input, then the general path (more than 16 tokens), the ReLU^2 form, and the refusal of a call
that needs more scratch than the built-in array holds."""
import numpy as np
import pytest
import torch

from oracle import qvb8_oracle as O
from qvb8_amd import _lib
from qvb8_amd.formats.qvb8 import pack as PK
from qvb8_amd.formats.qvb8.backends_experts import stack_projection
from qvb8_amd.formats.qvb8.module import QVBandLinearV8
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STATIC_BYTES = 2 * 1024 * 1024          # QVB8_MOE_STATIC_SCRATCH_BYTES of include/qvb8_amd.h


def _stack(E, hidden, inter, seed, gated=True):
    gu, dn = [], []
    for e in range(E):
        for lst, (Q, P) in ((gu, ((2 if gated else 1) * inter, hidden)), (dn, (hidden, inter))):
            enc = PK.encode_tensor(H.synth_weight(Q, P, seed=seed + 2 * e + len(lst)).to(DEV), 2e-3, restore="fp16")
            lst.append(QVBandLinearV8.from_encoded(enc))
    return stack_projection(gu), stack_projection(dn)


def _operands(stk, x, idx, w, act, out):
    g, d = stk
    T, k = idx.shape
    E = g["min_s"].shape[0]
    return [x.data_ptr(), _lib.dtype_code(x.dtype), T, idx.data_ptr(), w.data_ptr(), k, E,
            g["ids"].data_ptr(), g["ids"].numel(), g["min_s"].data_ptr(), g["tau_s"].data_ptr(), g["nbits"].data_ptr(),
            g["bit_off"].data_ptr(), g["Q"], g["P"],
            d["ids"].data_ptr(), d["ids"].numel(), d["min_s"].data_ptr(), d["tau_s"].data_ptr(), d["nbits"].data_ptr(),
            d["bit_off"].data_ptr(), d["Q"], d["P"], act, out.data_ptr(), _lib.dtype_code(out.dtype)]


def _both(lib, stk, T, k, seed, act=0, dtype=torch.bfloat16):
    g, d = stk
    E = g["min_s"].shape[0]
    act |= (0x100 if g["regular"] else 0) | (0x200 if d["regular"] else 0)      # what the operator states about its stacks
    rng = np.random.default_rng(seed)
    idx_h, w_h = O.router_topk(rng.normal(size=(T, E)), k)
    idx, w = torch.from_numpy(idx_h).to(DEV), torch.from_numpy(w_h).to(DEV)
    x = torch.randn(T, g["P"], generator=torch.Generator().manual_seed(seed)).to(dtype).to(DEV)
    need = lib.qvb8_moe_workspace_bytes(T, k, E, g["Q"], d["P"], d["Q"])
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    ref = torch.full((T, d["Q"]), float("nan"), dtype=dtype, device=DEV)
    got = torch.full((T, d["Q"]), float("nan"), dtype=dtype, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    _lib._check(lib.qvb8_moe_experts(*_operands(stk, x, idx, w, act, ref), ws.data_ptr(), ws.numel(), s), lib)
    rc = lib.qvb8_moe_experts_static(*_operands(stk, x, idx, w, act, got), s)
    return rc, need, ref, got


def test_static_scratch_matches_caller_workspace_twice_in_a_row():
    lib = _lib.load()
    stk = _stack(8, 512, 128, seed=40)
    # two calls in a row on the matrix-core path (up to 16 tokens), the second with a smaller input: what the first
    # call left in the shared array must not leak into the second
    for T, k, seed in ((12, 4, 1), (3, 2, 2)):
        rc, need, ref, got = _both(lib, stk, T, k, seed)
        assert rc == 0, lib.qvb8_last_error()
        assert need <= STATIC_BYTES
        torch.cuda.synchronize()
        assert not torch.isnan(ref.float()).any()
        assert torch.equal(ref.view(torch.int16), got.view(torch.int16)), (T, k)
    # the general path (plan + grouped products + combine), larger first, then smaller
    for T, k, seed in ((40, 4, 3), (17, 2, 4)):
        rc, need, ref, got = _both(lib, stk, T, k, seed, dtype=torch.float32)
        assert rc == 0, lib.qvb8_last_error()
        torch.cuda.synchronize()
        assert not torch.isnan(ref).any()
        assert torch.equal(ref.view(torch.int32), got.view(torch.int32)), (T, k)


def test_static_scratch_relu2_and_the_size_limit():
    lib = _lib.load()
    stk = _stack(4, 256, 128, seed=90, gated=False)
    rc, need, ref, got = _both(lib, stk, 5, 2, 7, act=1, dtype=torch.float16)
    assert rc == 0, lib.qvb8_last_error()
    torch.cuda.synchronize()
    assert torch.equal(ref.view(torch.int16), got.view(torch.int16))
    # a call whose workspace would not fit the built-in array is refused with a clear message and launches nothing
    T = 1200
    g, d = stk
    assert lib.qvb8_moe_workspace_bytes(T, 2, 4, g["Q"], d["P"], d["Q"]) > STATIC_BYTES
    rc, need, ref, got = _both(lib, stk, T, 2, 8, act=1, dtype=torch.float16)
    assert rc == -2 and b"scratch" in lib.qvb8_last_error()
    torch.cuda.synchronize()
    assert torch.isnan(got.float()).all()                   # untouched
