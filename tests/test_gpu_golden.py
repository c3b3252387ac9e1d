"""The HIP path against the committed known-answer fixtures of tests/golden, through the C ABI and
with no oracle in the loop.  Integer structures bit-exact; attention and dense layers within the
bf16 tolerance 2e-2 (outputs are bf16, references fp32)."""
import os

import numpy as np
import pytest
import torch

from tests.gpu_util import (DEV, n_bf16_bits, n_f16, n_u16, n_u32, t_bf16_bits, t_f16, t_u32)

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 2e-2


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


@pytest.mark.parametrize("rebalance", [0, 1])
@pytest.mark.parametrize("hash_op", [1, 2, 3, 4])
def test_psh_fixture(hash_op, rebalance):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import bucket as f3dbuck
    g = load("psh_256pts.npz")
    coords, seps = g["coords"].view(np.float16), g["seps"]
    nb, pad_to, n = int(g["num_bucket"]), int(g["pad_to"]), coords.shape[0]
    c, s = t_f16(coords), t_u32(seps)
    bucket_id = torch.ones(n, dtype=torch.uint16, device=DEV)
    cntr = torch.zeros(len(seps), nb, dtype=torch.uint32, device=DEV)
    offs = torch.empty(n, dtype=torch.uint32, device=DEV)
    cumsum = torch.zeros_like(cntr)
    scat = torch.full((pad_to, 3), float("nan"), dtype=torch.float16, device=DEV)
    bmin, bmax = torch.empty(3, dtype=torch.float16, device=DEV), torch.empty(3, dtype=torch.float16, device=DEV)
    pshattn.coord_bbox(c, bmin, bmax)
    mgr = pshattn.DeviceManagerSingleton.instance()
    mgr.init_dev_info(0)
    mgr.set_sync_stream(True)
    before = mgr.get_psh_rebalance()
    mgr.set_psh_rebalance(rebalance)
    try:
        pshattn.batch_psh_scatter_pad_hash(c, bucket_id, cntr, offs, s, int(g["max_n"]), nb, int(g["divisor"]),
                                           int(g["bucket_size"]), 0xFFFF, bmin, bmax,
                                           f3dbuck.generate_probe_offsets(DEV, shuffle_seed=0), cumsum, scat, 0.0, hash_op)
        torch.cuda.synchronize()
    finally:
        mgr.set_psh_rebalance(before)
    assert np.array_equal(n_f16(bmin).view(np.uint16), g["bbox_min"]) and np.array_equal(n_f16(bmax).view(np.uint16), g["bbox_max"])
    k = f"h{hash_op}_" + ("reb_" if rebalance else "")
    assert np.array_equal(n_u16(bucket_id), g[k + "ids"])
    assert np.array_equal(n_u32(cntr), g[k + "cnt"])
    assert np.array_equal(n_u32(offs), g[k + "off"])
    assert np.array_equal(n_u32(cumsum), g[k + "cumsum"])
    assert np.array_equal(n_f16(scat).view(np.uint16), g[k + "scat"])


@pytest.mark.parametrize("S", [2, 3])
def test_pool_fixture(S):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import subbuck
    g = load("pool_151pts.npz")
    coords, seps, feat = g["coords"].view(np.float16), g["seps"], g["feat"]
    c, s, f = t_f16(coords), t_u32(seps), t_bf16_bits(feat)
    k = f"s{S}_"
    for op in (0, 1, 2, 3):
        sb = subbuck.SubbuckBuffers.create_subbuck_buff(c, f, s, S, out_alignment=16)
        pshattn.batch_subbuck_reduce(c, f, s, 90, S, 0xFFFF, sb.bbox_min, sb.bbox_max, sb.subbuck_id, sb.subbuck_off,
                                     sb.reduced_sep, sb.reduced_coord, sb.reduced_feat, sb.unpool_ind, 1, op)
        torch.cuda.synchronize()
        assert np.array_equal(n_u32(sb.subbuck_id), g[k + "sub_id"]) and np.array_equal(n_u16(sb.subbuck_off), g[k + "sub_off"])
        assert np.array_equal(n_u32(sb.unpool_ind), g[k + "unpool"])
        assert np.array_equal(n_f16(sb.reduced_coord).view(np.uint16), g[k + "red_coord"])
        assert np.array_equal(n_u32(sb.reduced_sep), g[k + "red_sep"])
        assert np.array_equal(n_bf16_bits(sb.reduced_feat), g[k + f"red_op{op}"]), f"reduce op {op}"
    up = torch.zeros(feat.shape, dtype=torch.bfloat16, device=DEV)
    pshattn.additive_unpool_fwd(f, t_bf16_bits(g[k + "down"]), up, t_u32(g[k + "unpool"]), S)
    torch.cuda.synchronize()
    assert np.array_equal(n_bf16_bits(up), g[k + "up"])


@pytest.mark.parametrize("masked", [False, True])
def test_attention_fixture(masked):
    from flash3dtransformer_amd.lib import pshattn
    g = load("attn_2x128.npz")
    q, k, v = [t_bf16_bits(g[n]).reshape(1, 512, 2, 16) for n in "QKV"]
    O = torch.zeros_like(q)
    LSE = torch.zeros(1, 512, 2, dtype=torch.float32, device=DEV)
    kl = torch.from_numpy(g["kv_len"]).to(DEV) if masked else None
    pshattn.buck_swin_fwd(q, k, v, O, LSE, t_u32(g["scopes"]), int(g["bucket_size"]), kl)
    torch.cuda.synchronize()
    sfx = "_masked" if masked else ""
    assert np.abs(O.float().cpu().numpy() - g["O" + sfx]).max() <= TOL
    assert np.abs(LSE.cpu().numpy() - g["LSE" + sfx]).max() <= TOL


def test_dense_fixture():
    from flash3dtransformer_amd.lib import pshattn
    g = load("dense_64x32.npz")
    t = {n: t_bf16_bits(g[n]) for n in ("x", "ln_w", "ln_b", "w_qkv", "b_qkv", "w1", "b1", "w2", "b2")}
    new = lambda *s: torch.empty(*s, dtype=torch.bfloat16, device=DEV)
    ln, qkv, act, y = new(64, 32), new(64, 96), new(64, 64), new(64, 32)
    pshattn.layernorm_bf16(t["x"], t["ln_w"], t["ln_b"], ln, 1e-5)
    pshattn.ln_linear_bf16(t["x"], t["ln_w"], t["ln_b"], 1e-5, t["w_qkv"], t["b_qkv"], None, qkv, None)
    pshattn.ln_linear_bf16(t["x"], t["ln_w"], t["ln_b"], 1e-5, t["w1"], t["b1"], None, act, "swiglu")
    pshattn.linear_bf16(act, t["w2"], t["b2"], t["x"], y, None)
    torch.cuda.synchronize()
    for got, name in ((ln, "ln"), (qkv, "qkv"), (act, "act"), (y, "y")):
        want = g[name]
        err = np.abs(got.float().cpu().numpy() - want)
        assert err.max() <= TOL * max(1.0, np.abs(want).max()), f"{name}: max err {err.max()}"
