"""GPU parity at the full sizes of the benchmark configurations that the small-shape tests do not reach:
the 14B head count (H=40, model dim 5120; wan/configs/wan_t2v_14B.py:20-28), the reduce2xh tiling at 480p
(a=6, f=42, b1=15, b2=52) and one full-size attention block of each model against the same block code with
the oracle's operators on the CPU.  The oracle is evaluated on a few heads where all of them would take long."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import assert_close_16bit, max_abs, per_head_cosine, randn
from oracle import monarch, prologue
from oracle.ops import OracleOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H480, W480 = 30, 52
FRAME = H480 * W480


def test_prologue_at_the_14b_width():
    """One 1560-token frame at H=40, C=5120 (start_frame 18) against oracle.prologue: V rows bit-exact, q / k within
    one bf16 rounding step on a small fraction of elements (the mean of squares is summed in another order)."""
    H, D = 40, 128
    Cd, dtype = H * D, torch.bfloat16
    xq, xk, xv = (randn((1, FRAME, Cd), 800 + i, dtype) for i in range(3))
    wq, wk = (1 + 0.1 * randn((Cd,), 803)).to(dtype), (1 + 0.1 * randn((Cd,), 804)).to(dtype)
    q_o, k_o, v_o = prologue.qk_prologue(xq, xk, xv, wq, wk, H, (1, H480, W480), 18)
    kc = torch.zeros(1, 2 * FRAME, H, D, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    rope = sfa.prologue.rope_table(D, device=DEV)
    q = sfa.prologue.qk_prologue(xq.to(DEV), xk.to(DEV), xv.to(DEV), wq.to(DEV), wk.to(DEV), H, (1, H480, W480), 18, rope,
                                 kc, vc, FRAME)
    assert torch.equal(vc[:, FRAME:].cpu(), v_o) and not vc[:, :FRAME].any() and not kc[:, :FRAME].any()
    for got, ref in ((q, q_o), (kc[:, FRAME:], k_o)):
        diff = (got.float().cpu() - ref.float()).abs()
        assert (diff / ref.float().abs().clamp_min(1.0)).max().item() <= 2 * 2 ** -7          # one bf16 step
        assert (diff > 0).float().mean().item() < 1e-3


@pytest.mark.parametrize("heads_per_pass", [0, 8])
def test_monarch_op_with_40_heads(heads_per_pass):
    """The 14B op shape: H=40, a=3, f=21, b1=30, b2=52; oracle on heads 0, 17 and 39."""
    H, D, dtype = 40, 128, torch.bfloat16
    q = randn((1, 3 * FRAME, H, D), 810, dtype)
    k, v = randn((1, 21 * FRAME, H, D), 811, dtype), randn((1, 21 * FRAME, H, D), 812, dtype)
    out = sfa.monarch_attn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, H480, W480, heads_per_pass=heads_per_pass,
                                        kv_block_order=True)
    heads = [0, 17, 39]
    ref = monarch.monarch_attn(q[:, :, heads], k[:, :, heads], v[:, :, heads], 1, 1, 1, H480, W480, dtype=torch.float32)
    assert_close_16bit(out[:, :, heads], ref, dtype)
    assert torch.isfinite(out.float()).all()


def test_kv_cache_op_at_the_reduce2xh_shape():
    """configs[3] op shape: 12 heads, h_reduce = 2 (a=6, f=42, b1=15, b2=52), chunk written at frames 18..20; the
    cache rows bit for bit, the output against the oracle on heads 3 and 11."""
    H, D, dtype = 12, 128, torch.bfloat16
    tiling = (1, 2, 1)
    q, nk, nv = (randn((1, 3 * FRAME, H, D), 820 + i, dtype) for i in range(3))
    kc, vc = randn((1, 21 * FRAME, H, D), 823, dtype), randn((1, 21 * FRAME, H, D), 824, dtype)
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = sfa.monarch_attn.monarch_attn_with_kv_cache(q.to(DEV), kd, vd, nk.to(DEV), nv.to(DEV), 18 * FRAME, 21 * FRAME, *tiling,
                                                      H480, W480)
    heads = [3, 11]
    kc_o, vc_o = kc[:, :, heads].clone(), vc[:, :, heads].clone()
    ref = monarch.monarch_attn_with_kv_cache(q[:, :, heads], kc_o, vc_o, nk[:, :, heads], nv[:, :, heads], 18 * FRAME, 21 * FRAME,
                                             *tiling, H480, W480, dtype=torch.float32)
    assert torch.equal(kd[:, :, heads].cpu(), kc_o) and torch.equal(vd[:, :, heads].cpu(), vc_o)
    assert_close_16bit(out[:, :, heads], ref, dtype)


@pytest.mark.parametrize("name", ["1.3B", "14B"])
def test_one_full_size_block_against_oracle_operators(name):
    """One CausalWanAttentionBlock at the model's real width: 4680 tokens (frames 18..20) against a cache that holds
    18 frames; the GPU run (HIP operators) against the same module code on the CPU with the oracle's operators.
    bf16 GEMMs accumulate in another order on the two sides: cosine > 0.999 and max-abs below 3 % of the range."""
    cm = sfa.causal_model
    cfg = cm.WAN_CONFIGS[name]
    dim, heads = cfg["dim"], cfg["num_heads"]
    dtype = torch.bfloat16
    torch.manual_seed(7)
    ref = cm.CausalWanAttentionBlock(dim, cfg["ffn_dim"], heads, block_num=0, ops=OracleOps(),
                                     flags=cm.AttentionFlags(0, use_framewise=True))
    for m in ref.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.xavier_uniform_(m.weight)
            torch.nn.init.normal_(m.bias, std=0.02)
    ref = ref.to(dtype).eval()
    dev = cm.CausalWanAttentionBlock(dim, cfg["ffn_dim"], heads, block_num=0,
                                     flags=cm.AttentionFlags(0, use_framewise=True)).to(dtype).eval()
    dev.load_state_dict(ref.state_dict())
    dev = dev.to(DEV)

    x = randn((1, 3 * FRAME, dim), 830, dtype)
    e = (0.3 * randn((1, 3, 6, dim), 831)).to(dtype)
    ctx = randn((1, 512, dim), 832, dtype)
    k0, v0 = randn((1, 21 * FRAME, heads, 128), 833, dtype), randn((1, 21 * FRAME, heads, 128), 834, dtype)

    def cache(device):
        return {"k": k0.clone().to(device), "v": v0.clone().to(device),
                "global_end_index": torch.tensor([18 * FRAME], device=device),
                "local_end_index": torch.tensor([18 * FRAME], device=device)}

    kv_r, kv_d = cache("cpu"), cache(DEV)
    ca_r, ca_d = ({"k": None, "v": None, "is_init": False} for _ in range(2))
    with torch.no_grad():
        y_ref = ref(x, e, (3, H480, W480), ctx, kv_r, ca_r, 18 * FRAME)
        y_dev = dev(x.to(DEV), e.to(DEV), (3, H480, W480), ctx.to(DEV), kv_d, ca_d, 18 * FRAME)
    assert kv_d["_global_end"] == 21 * FRAME and kv_d["_local_end"] == 21 * FRAME
    assert torch.equal(kv_d["v"].cpu()[:, :18 * FRAME], v0[:, :18 * FRAME])           # old rows untouched
    assert max_abs(kv_d["k"][:, 18 * FRAME:], kv_r["k"][:, 18 * FRAME:]) <= 2 ** -4       # new rows: GEMM + prologue rounding
    cos = torch.nn.functional.cosine_similarity(y_dev.double().flatten().cpu(), y_ref.double().flatten(), dim=0).item()
    assert cos > 0.999, cos
    assert max_abs(y_dev, y_ref) < 0.03 * y_ref.float().abs().max().item()
    # the attention sub-layer alone, on identical inputs: the reference's bar
    q = randn((1, 3 * FRAME, heads, 128), 835, dtype)
    hsel = [0, heads - 1]
    o_dev = sfa.monarch_attn.monarch_attn(q.to(DEV), kv_d["k"], kv_d["v"], 1, 1, 1, H480, W480, kv_block_order=True)
    kr, vr = kv_d["k"].cpu(), kv_d["v"].cpu()
    o_ref = monarch.monarch_attn(q[:, :, hsel], kr[:, :, hsel], vr[:, :, hsel], 1, 1, 1, H480, W480, dtype=torch.float32)
    assert_close_16bit(o_dev[:, :, hsel], o_ref, dtype)
    assert per_head_cosine(o_dev[:, :, hsel], o_ref) > 0.999
