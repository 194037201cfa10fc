"""Every entry point refuses malformed requests with the documented status code and a message that
names the problem, before anything is enqueued.

The pointers handed in are addresses inside a host buffer (never dereferenced: each case fails an
argument check first), and the whole module is skipped where a GPU is present, so that no case can
reach a launch with them whatever a later change does to the order of the checks."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.skipif(torch.cuda.is_available(), reason="runs on GPU-less hosts only")

EINVAL, EUNSUPPORTED = -1, -2


@pytest.fixture(scope="module")
def env():
    from kfold_amd import _lib

    lib = _lib.lib()
    buf = ctypes.create_string_buffer(1 << 16)
    base = ctypes.addressof(buf)
    p = [base + 4096 * i for i in range(12)]          # distinct non-null addresses
    return lib, p, buf


def _expect(lib, rc, code, *words):
    msg = lib.kfh_last_error().decode()
    assert rc == code, (rc, msg)
    for w in words:
        assert w in msg, msg


def test_trimul_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_trimul_workspace_bytes(64, 128)
    f = lib.kfh_trimul_forward
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 80, 0, 1e-5, 0, None), EUNSUPPORTED, "C=80")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 0, 64, 128, 0, 1e-5, 0, None), EINVAL, "B=0")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, -3, 128, 0, 1e-5, 0, None), EINVAL, "N=-3")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 128, 0, 1e-5, 7, None), EINVAL, "io_dtype 7")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 128, 2, 1e-5, 0, None), EINVAL, "direction 2")
    _expect(lib, f(p[0], None, p[2], None, p[3], p[4], need, 1, 64, 128, 0, 1e-5, 0, None), EINVAL, "null")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], None, need, 1, 64, 128, 0, 1e-5, 0, None), EINVAL, "null")
    # writing over z is allowed only as the fused in-place update z += f(z)
    _expect(lib, f(p[0], p[1], p[2], None, p[0], p[4], need, 1, 64, 128, 0, 1e-5, 0, None), EINVAL, "alias")
    _expect(lib, f(p[0], p[1], p[2], p[5], p[0], p[4], need, 1, 64, 128, 0, 1e-5, 0, None), EINVAL, "alias")
    _expect(lib, f(p[0], p[1], p[2], p[0], p[0], p[4], need - 1, 1, 64, 128, 0, 1e-5, 0, None), EINVAL,
            "workspace", str(need))
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], 0, 1, 64, 256, 1, 1e-5, 1, None), EINVAL, "workspace")
    g = lib.kfh_trimul_pack
    _expect(lib, g(*p[:8], 0, 48, p[8], None), EUNSUPPORTED, "C=48")
    _expect(lib, g(*p[:8], 5, 128, p[8], None), EINVAL, "w_dtype 5")
    _expect(lib, g(*p[:7], None, 0, 128, p[8], None), EINVAL, "null")
    _expect(lib, g(*p[:8], 0, 128, None, None), EINVAL, "null")
    # the stage-selective variant checks the same things
    s = lib.kfh_trimul_forward_stages
    _expect(lib, s(p[0], p[1], p[2], None, p[3], p[4], 0, 1, 64, 128, 0, 1e-5, 0, 7, None), EINVAL, "workspace")
    # ranges of rows: tile-aligned, one batch element, the fused widths
    r = lib.kfh_trimul_forward_rows
    assert lib.kfh_trimul_row_granule(768, 128) == 256 and lib.kfh_trimul_row_granule(300, 256) == 128
    assert lib.kfh_trimul_row_granule(300, 64) == 0 and lib.kfh_trimul_row_granule(0, 128) == 0
    big = lib.kfh_trimul_workspace_bytes(768, 128)
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 128, 0, 1e-5, 0, 6, 100, 256, None), EINVAL,
            "multiples of 256")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 128, 0, 1e-5, 0, 6, 256, 100, None), EINVAL, "rows [256, 356)")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 128, 0, 1e-5, 0, 6, 512, 512, None), EINVAL, "of 768")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 2, 768, 128, 0, 1e-5, 0, 6, 0, 256, None), EUNSUPPORTED, "B = 1")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 64, 0, 1e-5, 0, 6, 0, 256, None), EUNSUPPORTED, "C = 128 or 256")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], 0, 1, 768, 128, 0, 1e-5, 0, 6, 256, 512, None), EINVAL, "workspace")


def test_triattn_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_triattn_workspace_bytes(64, 128, 4)
    assert need > 0 and lib.kfh_triattn_workspace_bytes(64, 64, 4) > 0
    assert lib.kfh_triattn_workspace_bytes(9000, 128, 4) == 0 and lib.kfh_triattn_workspace_bytes(64, 100, 4) == 0
    f = lib.kfh_triattn_forward
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 100, 4, 0, 1e-5, 0, None), EUNSUPPORTED, "C=100")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 128, 1, 0, 1e-5, 0, None), EUNSUPPORTED, "H=1")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 9000, 128, 4, 0, 1e-5, 0, None), EUNSUPPORTED, "8192")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, -1, 64, 128, 4, 0, 1e-5, 0, None), EINVAL, "B=-1")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], need, 1, 64, 128, 4, 0, 1e-5, 3, None), EINVAL, "io_dtype")
    _expect(lib, f(None, p[1], p[2], None, p[3], p[4], need, 1, 64, 128, 4, 0, 1e-5, 0, None), EINVAL, "null")
    _expect(lib, f(p[0], p[1], p[2], None, p[0], p[4], need, 1, 64, 128, 4, 1, 1e-5, 0, None), EINVAL, "alias")
    _expect(lib, f(p[0], p[1], p[2], p[0], p[0], p[4], need - 1, 1, 64, 128, 4, 1, 1e-5, 0, None), EINVAL, "workspace")
    _expect(lib, f(p[0], p[1], p[2], None, p[3], p[4], 16, 2, 64, 64, 4, 0, 1e-5, 0, None), EINVAL, "workspace")
    r = lib.kfh_triattn_forward_rows
    big = lib.kfh_triattn_workspace_bytes(768, 128, 4)
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 128, 4, 0, 1e-5, 0, 6, 700, 100, None), EINVAL, "rows [700, 800)")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 128, 4, 0, 1e-5, 0, 6, -1, 100, None), EINVAL, "rows")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 2, 768, 128, 4, 0, 1e-5, 0, 6, 0, 100, None), EUNSUPPORTED, "B = 1")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], big, 1, 768, 64, 4, 0, 1e-5, 0, 6, 0, 100, None), EUNSUPPORTED, "C = 128")
    _expect(lib, r(p[0], p[1], p[2], None, p[3], p[4], 0, 1, 768, 128, 4, 0, 1e-5, 0, 6, 0, 100, None), EINVAL, "workspace")
    g = lib.kfh_triattn_pack
    _expect(lib, g(*p[:8], 0, 128, 3, p[8], None), EUNSUPPORTED, "H=3")
    _expect(lib, g(*p[:8], 9, 128, 4, p[8], None), EINVAL, "w_dtype")
    _expect(lib, g(*p[:2], None, *p[3:8], 0, 128, 4, p[8], None), EINVAL, "null")


def test_transition_and_bias_argument_checks(env):
    lib, p, _ = env
    f = lib.kfh_transition_forward
    _expect(lib, f(p[0], p[1], None, None, p[2], None, 0, 10, 100, 4, 1e-5, 0, None), EUNSUPPORTED, "C=100")
    _expect(lib, f(p[0], p[1], None, None, p[2], None, 0, 10, 128, 9, 1e-5, 0, None), EUNSUPPORTED, "E=9")
    _expect(lib, f(p[0], p[1], None, None, p[2], None, 0, -1, 128, 2, 1e-5, 0, None), EINVAL, "rows=-1")
    _expect(lib, f(p[0], p[1], None, None, p[2], None, 0, 10, 128, 2, 1e-5, 4, None), EINVAL, "io_dtype")
    _expect(lib, f(None, p[1], None, None, p[2], None, 0, 10, 128, 2, 1e-5, 0, None), EINVAL, "null")
    # token-track widths need the workspace (the fused C = 128 / 256 kernels do not)
    need = lib.kfh_transition_workspace_bytes(10, 384, 4)
    assert lib.kfh_transition_workspace_bytes(10, 256, 4) == 0 and lib.kfh_transition_workspace_bytes(10, 64, 2) > 0
    _expect(lib, f(p[0], p[1], None, None, p[2], p[4], need - 1, 10, 384, 4, 1e-5, 0, None), EINVAL, "workspace")
    _expect(lib, f(p[0], p[1], None, None, p[2], None, 0, 10, 384, 4, 1e-5, 0, None), EINVAL)
    g = lib.kfh_transition_pack
    _expect(lib, g(p[0], p[1], p[2], p[3], 0, 130, 4, p[4], None), EUNSUPPORTED, "C=130")
    _expect(lib, g(p[0], p[1], None, p[3], 0, 128, 2, p[4], None), EINVAL, "null")
    # pair bias projection and dense -> tiles
    assert lib.kfh_pair_bias_packed_bytes(128, 16) > 0 and lib.kfh_pair_bias_packed_bytes(128, 33) == 0
    assert lib.kfh_pair_bias_packed_bytes(256, 16) == 0
    _expect(lib, lib.kfh_pair_bias_pack(p[0], p[1], p[2], 0, 256, 16, p[3], None), EUNSUPPORTED, "C=256")
    _expect(lib, lib.kfh_pair_bias_pack(p[0], p[1], None, 0, 128, 16, p[3], None), EINVAL)
    _expect(lib, lib.kfh_pair_bias_project(p[0], p[1], p[2], 1, 64, 128, 40, 1e-5, 0, None), EUNSUPPORTED, "H=40")
    _expect(lib, lib.kfh_pair_bias_project(None, p[1], p[2], 1, 64, 128, 16, 1e-5, 0, None), EINVAL)
    _expect(lib, lib.kfh_pair_bias_project(p[0], p[1], p[2], 1, 0, 128, 16, 1e-5, 0, None), EINVAL)
    assert lib.kfh_bias_tiles_bytes(2, 16, 100, 0) == 2 * 16 * 4 * 4 * 2048       # 4 x 4 blocks of 2 KiB
    assert lib.kfh_bias_tiles_bytes(2, 16, 100, 1) == 2 * 16 * 4 * 4 * 4096       # fp32 tiles
    assert lib.kfh_bias_tiles_bytes(2, 16, 100, 2) == 0
    _expect(lib, lib.kfh_bias_tiles_from_dense(None, 0, p[0], 1, 16, 100, 0, None), EINVAL)
    _expect(lib, lib.kfh_bias_tiles_from_dense(p[0], 2, p[1], 1, 16, 100, 0, None), EINVAL, "io_dtype")
    _expect(lib, lib.kfh_bias_tiles_from_dense(p[0], 0, p[1], 1, 16, 100, 7, None), EINVAL, "arith")


def test_pair_bias_attention_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_apb_workspace_bytes(2, 100, 384, 16, 0, 0)
    assert need > 0 and lib.kfh_apb_workspace_bytes(2, 100, 384, 5, 0, 0) == 0    # head dim 76.8
    assert lib.kfh_apb_workspace_bytes(2, 100, 384, 2, 0, 0) == 0                 # head dim 192 > 64
    # fp32 arithmetic: three bf16 parts of everything
    assert lib.kfh_apb_workspace_bytes(2, 100, 384, 16, 0, 1) > 2 * need
    assert lib.kfh_apb_workspace_bytes(2, 100, 384, 16, 0, 2) == 0
    assert lib.kfh_apb_packed_bytes(384, 16, 0, 1) > 2 * lib.kfh_apb_packed_bytes(384, 16, 0, 0)
    f = lib.kfh_apb_forward

    def call(a=p[0], s=None, tiles=p[1], mask=p[2], blob=p[3], res=None, out=p[4], ws=p[5], ws_bytes=need,
             S=2, L=100, C=384, H=16, Cs=0, norm=1, eps=1e-5, io=0, arith=0):
        return f(a, s, tiles, mask, blob, res, out, ws, ws_bytes, S, L, C, H, Cs, norm, 0, 0, 0, eps, io, arith,
                 None)

    _expect(lib, call(arith=3), EUNSUPPORTED, "arith=3")
    _expect(lib, call(arith=1), EINVAL, "workspace")          # the bf16 workspace size is too small for fp32
    _expect(lib, call(C=400), EUNSUPPORTED, "C=400")
    _expect(lib, call(H=5), EUNSUPPORTED, "H=5")
    _expect(lib, call(S=0), EINVAL, "S=0")
    _expect(lib, call(L=9000), EUNSUPPORTED, "8192")
    _expect(lib, call(io=2), EINVAL, "io_dtype")
    _expect(lib, call(tiles=None), EINVAL, "null")
    _expect(lib, call(Cs=384, C=768, H=16, s=None, ws_bytes=1 << 40), EINVAL, "s_cond")
    _expect(lib, call(ws_bytes=need - 1), EINVAL, "workspace", str(need))
    g = lib.kfh_apb_pack
    w = p[:8]
    _expect(lib, g(*w, None, None, None, None, None, None, 0, 384, 7, 0, 0, p[8], None), EUNSUPPORTED, "H=7")
    _expect(lib, g(*w, None, None, None, None, None, None, 3, 384, 16, 0, 0, p[8], None), EINVAL, "w_dtype")
    _expect(lib, g(*w[:2], None, *w[3:], None, None, None, None, None, None, 0, 384, 16, 0, 0, p[8], None), EINVAL, "null")
    _expect(lib, g(*w, None, None, None, None, None, None, 0, 768, 16, 384, 0, p[8], None), EINVAL, "AdaLN")
    _expect(lib, g(*w, None, None, None, None, None, None, 0, 384, 16, 0, 5, p[8], None), EUNSUPPORTED, "arith=5")


def test_window_attention_and_recurrence_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_cross_apb_workspace_bytes(6, 32, 128, 128, 4, 0, 0)
    assert lib.kfh_cross_apb_workspace_bytes(6, 32, 128, 128, 4, 0, 1) > 2 * need
    f = lib.kfh_cross_apb_forward

    def call(aq=p[0], ak=p[1], sq=None, sk=None, bias=p[2], bdt=0, mask=p[3], blob=p[4], res=None, out=p[5],
             ws=p[6], ws_bytes=need, W=6, Lq=32, Lk=128, C=128, H=4, Cs=0, io=0, norm=1, arith=0):
        return f(aq, ak, sq, sk, bias, bdt, mask, blob, res, out, ws, ws_bytes, W, Lq, Lk, C, H, Cs, norm, 1e-5,
                 io, arith, None)

    _expect(lib, call(arith=4), EUNSUPPORTED, "arith=4")
    _expect(lib, call(C=100), EUNSUPPORTED, "C=100")
    _expect(lib, call(W=0), EINVAL, "W=0")
    _expect(lib, call(Lk=10000), EUNSUPPORTED, "10000")
    _expect(lib, call(bdt=9), EINVAL, "dtype")
    _expect(lib, call(ak=None), EINVAL, "null")
    _expect(lib, call(Cs=64, ws_bytes=1 << 40), EINVAL, "s_q")
    _expect(lib, call(ws_bytes=need - 1), EINVAL, "workspace")
    g = lib.kfh_parcae_step
    _expect(lib, g(p[0], p[1], None, p[2], p[3], 10, 192, 1e-5, 0, None), EUNSUPPORTED, "C=192")
    _expect(lib, g(p[0], p[1], None, p[2], p[3], -1, 128, 1e-5, 0, None), EINVAL, "rows=-1")
    _expect(lib, g(p[0], p[1], None, p[2], p[3], 10, 128, 1e-5, 5, None), EINVAL, "io_dtype")
    _expect(lib, g(p[0], None, None, p[2], p[3], 10, 128, 1e-5, 0, None), EINVAL, "null")
    # the step may run in place on the state, never over its inputs
    _expect(lib, g(p[0], p[1], None, p[2], p[1], 10, 128, 1e-5, 0, None), EINVAL, "alias")
    _expect(lib, g(p[0], p[1], p[4], p[2], p[4], 10, 128, 1e-5, 0, None), EINVAL, "alias")
    h = lib.kfh_parcae_pack
    _expect(lib, h(p[0], p[1], p[2], p[3], p[4], 0, 64, p[5], None), EUNSUPPORTED, "C=64")
    _expect(lib, h(p[0], p[1], None, p[3], p[4], 0, 128, p[5], None), EINVAL, "null")


def test_pair_block_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_pair_block_workspace_bytes(1, 64, 128, 4, 2)
    assert need == max(lib.kfh_trimul_workspace_bytes(64, 128), lib.kfh_triattn_workspace_bytes(64, 128, 4))
    assert lib.kfh_pair_block_workspace_bytes(3, 40, 64, 4, 2) >= lib.kfh_triattn_workspace_bytes_batched(3, 40, 64, 4)
    assert lib.kfh_pair_block_workspace_bytes(0, 64, 128, 4, 2) == 0
    f = lib.kfh_pair_block_forward
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], need, 1, 64, 48, 4, 2, 1e-5, 0, None), EUNSUPPORTED, "C=48")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], need, 1, 64, 128, 3, 2, 1e-5, 0, None), EUNSUPPORTED, "H=3")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], need, 0, 64, 128, 4, 2, 1e-5, 0, None), EINVAL, "B=0")
    _expect(lib, f(p[0], p[1], p[2], p[3], None, p[5], p[6], p[7], need, 1, 64, 128, 4, 2, 1e-5, 0, None), EINVAL, "null")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], need - 1, 1, 64, 128, 4, 2, 1e-5, 0, None), EINVAL,
            "workspace", str(need))
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], need, 1, 64, 128, 4, 2, 1e-5, 9, None), EINVAL, "io_dtype")


def test_single_track_argument_checks(env):
    lib, p, _ = env
    need = lib.kfh_single_track_workspace_bytes(1, 64, 128, 384, 16, 4)
    assert need >= lib.kfh_bias_tiles_bytes(1, 16, 64, 0) + lib.kfh_apb_workspace_bytes(1, 64, 384, 16, 0, 0)
    assert lib.kfh_single_track_workspace_bytes(1, 64, 256, 384, 16, 4) == 0       # pair bias is built for c_z = 128
    f = lib.kfh_single_track_forward
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], need, 1, 64, 256, 384, 16, 4, 1e-5, 0, None), EUNSUPPORTED, "Cz=256")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], need, 1, 64, 128, 384, 5, 4, 1e-5, 0, None), EUNSUPPORTED, "H=5")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], need, 0, 64, 128, 384, 16, 4, 1e-5, 0, None), EINVAL, "B=0")
    _expect(lib, f(p[0], None, p[2], p[3], p[4], p[5], p[6], need, 1, 64, 128, 384, 16, 4, 1e-5, 0, None), EINVAL, "null")
    _expect(lib, f(p[0], p[1], p[2], p[3], p[4], p[5], p[6], need - 1, 1, 64, 128, 384, 16, 4, 1e-5, 0, None), EINVAL,
            "workspace", str(need))
