"""GPU parity of the fused recurrent kernel (decode path) against the CPU oracle and against the chunked path."""
import pytest
import torch

from hdla_hip import chunk_hrdplr_delta_rule, fused_recurrent_dplr_delta_rule
from hdla_hip.synthetic import make_config, make_inputs
from oracle import hrdplr_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _run(inp, dtype, **kw):
    t = [x.to(dtype).to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    return fused_recurrent_dplr_delta_rule(*t, 2, **kw)


def _ref(inp, dtype, **kw):
    t = [x.to(dtype) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    return O.recurrence(*t, kw.pop("scale"), kw.pop("initial_state", None), **kw)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 5e-3)])
@pytest.mark.parametrize("B,T,H,K,V", [(2, 37, 2, 64, 64), (1, 20, 3, 128, 128), (2, 9, 2, 64, 128), (1, 5, 2, 128, 64)])
def test_parity(dtype, tol, B, T, H, K, V):
    inp = make_inputs(200 + T, B, T, H, K, V, gk_div=1.0)
    o, ht = _run(inp, dtype, scale=0.5, initial_state=inp.h0.to(DEV), output_final_state=True)
    o_r, ht_r = _ref(inp, dtype, scale=0.5, initial_state=inp.h0)
    assert o.dtype == dtype and ht.dtype == torch.float32
    assert O.rel_l2(o, o_r) <= tol and O.rel_l2(ht, ht_r) <= min(tol, 1e-5)


def test_reverse_varlen_and_no_state():
    inp = make_inputs(31, 1, 60, 2, 64, 64, n_states=3)
    cu = torch.tensor([0, 11, 40, 60])
    o, ht = _run(inp, torch.float32, scale=1.0, initial_state=inp.h0.to(DEV), output_final_state=True, reverse=True,
                 cu_seqlens=cu.to(DEV))
    o_r, ht_r = _ref(inp, torch.float32, scale=1.0, initial_state=inp.h0, reverse=True, cu_seqlens=cu)
    assert O.rel_l2(o, o_r) <= 1e-5 and O.rel_l2(ht, ht_r) <= 1e-5
    o, ht = _run(inp, torch.float32)                                         # defaults: no state in or out
    o_r, _ = _ref(inp, torch.float32, scale=64 ** -0.5)
    assert ht is None and O.rel_l2(o, o_r) <= 1e-5


def test_matches_chunked_entry():
    """The reference's own cross check (test_recurrent.py:66-67): chunk output == recurrent output, final states too."""
    inp = make_inputs(32, 2, 256, 4, 128, 64, gk_div=1.0)
    t = [x.float().to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    h0 = inp.h0.to(DEV)
    o1, h1 = chunk_hrdplr_delta_rule(*t, 2, scale=1.0, initial_state=h0, output_final_state=True, chunk_size=16)
    o2, h2 = fused_recurrent_dplr_delta_rule(*t, 2, scale=1.0, initial_state=h0, output_final_state=True)
    assert O.rel_l2(o1, o2) <= 1e-5 and O.rel_l2(h1, h2) <= 1e-5


def test_decode_steps_config4_reduced():
    """Configuration 4's loop at B = 8, H = 4: 16 single-token calls carrying the fp32 state, against one
    16-token oracle run."""
    steps = 16
    inp = make_config(4, shape=(8, steps, 4, 128, 128))
    t = [x.bfloat16().to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    q, k, v, a, b, gk = t
    S = inp.h0.to(DEV)
    outs = []
    for i in range(steps):
        o, S = fused_recurrent_dplr_delta_rule(q[:, i:i + 1], k[:, i:i + 1], v[:, i:i + 1], a[:, 2 * i:2 * i + 2],
                                               b[:, 2 * i:2 * i + 2], gk[:, i:i + 1], 2, scale=1.0, initial_state=S,
                                               output_final_state=True)
        outs.append(o)
    o = torch.cat(outs, 1)
    o_r, S_r = O.recurrence(*[x.bfloat16() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)], 1.0, inp.h0)
    assert O.rel_l2(o, o_r) <= 5e-3 and O.rel_l2(S, S_r) <= 1e-5


def test_decode_steps_config4_full_size_batch_subset():
    """Configuration 4 at full size (B256 H32 K=V=128 bf16 inputs, fp32 state of 512 MiB): 64 single-token calls
    carrying the state; the CPU oracle runs the same 64 tokens for three of the 256 sequences."""
    steps = 64
    inp = make_config(4, shape=(256, steps, 32, 128, 128))
    t = [x.bfloat16().to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    q, k, v, a, b, gk = t
    S = inp.h0.to(DEV)
    outs = []
    for i in range(steps):
        o, S = fused_recurrent_dplr_delta_rule(q[:, i:i + 1], k[:, i:i + 1], v[:, i:i + 1], a[:, 2 * i:2 * i + 2],
                                               b[:, 2 * i:2 * i + 2], gk[:, i:i + 1], 2, scale=1.0, initial_state=S,
                                               output_final_state=True)
        outs.append(o)
    o = torch.cat(outs, 1)
    assert torch.isfinite(o.float()).all() and torch.isfinite(S).all()
    sel = [0, 101, 255]
    o_r, S_r = O.recurrence(*[x[sel].bfloat16() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)], 1.0, inp.h0[sel])
    e_o, e_s = O.rel_l2(o[sel], o_r), O.rel_l2(S[sel], S_r)
    print(f"cfg4 full size, 64 carried steps: o {e_o:.2e} state {e_s:.2e}", flush=True)
    assert e_o <= 5e-3 and e_s <= 1e-5


def test_decode_config4_full_size_all_1024_carried_steps():
    """Configuration 4 exactly as it is timed: B256 H32 K=V=128, bf16 inputs, 1024 single-token calls carrying the fp32
    state.  The inputs are drawn on the GPU in blocks of 64 steps (the whole run's inputs would be 40 GB on the host);
    the CPU oracle runs all 1024 tokens for two of the 256 sequences."""
    import torch.nn.functional as F
    B, H, K, V, steps, blk = 256, 32, 128, 128, 1024, 64
    sel = [3, 200]
    g = torch.Generator(device=DEV).manual_seed(4004)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV, dtype=torch.float32)
    S = rn(B, H, K, V) * 0.1
    S0 = S[sel].cpu()
    kept = {n: [] for n in ("q", "k", "v", "a", "b", "gk")}
    outs = []
    for j in range(steps // blk):
        q, k, v = F.normalize(rn(B, blk, H, K), dim=-1), F.normalize(rn(B, blk, H, K), dim=-1), rn(B, blk, H, V)
        b_r = [F.normalize(rn(B, blk, H, K), dim=-1) for _ in range(2)]
        a_r = [-2.0 * torch.rand(B, blk, H, 1, generator=g, device=DEV) * bb for bb in b_r]
        a = torch.stack(a_r, dim=2).reshape(B, 2 * blk, H, K)
        b = torch.stack(b_r, dim=2).reshape(B, 2 * blk, H, K)
        gk = F.logsigmoid(rn(B, blk, H, K)) / 16
        t = dict(q=q.bfloat16(), k=k.bfloat16(), v=v.bfloat16(), a=a.bfloat16(), b=b.bfloat16(), gk=gk.bfloat16())
        for n in kept:
            kept[n].append(t[n][sel].cpu())
        for i in range(blk):
            o, S = fused_recurrent_dplr_delta_rule(t["q"][:, i:i + 1], t["k"][:, i:i + 1], t["v"][:, i:i + 1],
                                                   t["a"][:, 2 * i:2 * i + 2], t["b"][:, 2 * i:2 * i + 2], t["gk"][:, i:i + 1],
                                                   2, scale=1.0, initial_state=S, output_final_state=True)
            outs.append(o[sel])
        del q, k, v, a, b, gk, t
    o = torch.cat(outs, 1)
    assert torch.isfinite(S).all()
    ref = [torch.cat(kept[n], 1) for n in ("q", "k", "v", "a", "b", "gk")]
    o_r, S_r = O.recurrence(*ref, 1.0, S0)
    e_o, e_s = O.rel_l2(o, o_r), O.rel_l2(S[sel], S_r)
    print(f"cfg4 full size, 1024 carried steps: o {e_o:.2e} state {e_s:.2e}", flush=True)
    assert e_o <= 5e-3 and e_s <= 1e-5


def test_rank_one_and_padded_dims():
    inp = make_inputs(33, 2, 12, 2, 96, 48, R=1)
    t = [x.float().to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    o, ht = fused_recurrent_dplr_delta_rule(*t, 1, scale=1.0, initial_state=inp.h0.to(DEV), output_final_state=True)
    o_r, ht_r = O.recurrence(inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk, 1.0, inp.h0, rank_ab=1)
    assert o.shape == (2, 12, 2, 48) and ht.shape == (2, 2, 96, 48)
    assert O.rel_l2(o, o_r) <= 1e-5 and O.rel_l2(ht, ht_r) <= 1e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 5e-3)])
@pytest.mark.parametrize("K,V", [(256, 256), (200, 72), (64, 256), (256, 128)])
def test_head_sizes_up_to_256(dtype, tol, K, V):
    """The reference's token-serial kernel takes any K (BK = next_pow2(K), recurrent.py:155-176); here up to 256, both
    operators (a, b given; a, b formed in the kernel), with a packed batch."""
    from hdla_hip import fused_recurrent_hdla_delta_rule
    inp = make_inputs(700 + K + V, 1, 23, 2, K, V, gk_div=2.0, n_states=2)
    cu = torch.tensor([0, 9, 23])
    o, ht = _run(inp, dtype, scale=0.5, initial_state=inp.h0.to(DEV), output_final_state=True, cu_seqlens=cu.to(DEV))
    o_r, ht_r = _ref(inp, dtype, scale=0.5, initial_state=inp.h0, cu_seqlens=cu)
    assert o.shape == inp.v.shape and ht.shape == inp.h0.shape
    assert O.rel_l2(o, o_r) <= tol and O.rel_l2(ht, ht_r) <= min(tol, 1e-5)
    g = torch.Generator().manual_seed(1)
    beta = 2 * torch.rand(1, 23, 2, 1, generator=g)
    q, k, v, lf = (x.to(dtype) for x in (inp.q, inp.k, inp.v, inp.gk))
    o2, h2 = fused_recurrent_hdla_delta_rule(q.to(DEV), k.to(DEV), v.to(DEV), beta.to(dtype).to(DEV), lf.to(DEV), scale=1.0,
                                             initial_state=inp.h0[:1].to(DEV), output_final_state=True)
    a, b = O.parameterize_a_b(beta.to(dtype).double(), k.double(), lf.double())
    o2_r, h2_r = O.recurrence(q, k, v, a.to(dtype), b.to(dtype), lf, 1.0, inp.h0[:1])
    assert O.rel_l2(o2, o2_r) <= tol and O.rel_l2(h2, h2_r) <= min(tol, 1e-5)


def test_chunked_operator_refuses_what_only_the_token_serial_one_takes():
    """Head dimensions above 128: the chunked operator raises a ValueError that names the token-serial operator, and
    that operator runs the same inputs (checked against the float64 recurrence)."""
    inp = make_inputs(77, 1, 24, 2, 256, 192)
    t = [x.bfloat16().to(DEV) for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    with pytest.raises(ValueError, match="fused_recurrent_dplr_delta_rule"):
        chunk_hrdplr_delta_rule(*t, 2, scale=1.0, initial_state=inp.h0.to(DEV), output_final_state=True)
    o, ht = fused_recurrent_dplr_delta_rule(*t, 2, scale=1.0, initial_state=inp.h0.to(DEV), output_final_state=True)
    o_r, ht_r = O.recurrence(*[x.bfloat16() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)], 1.0, inp.h0)
    assert O.rel_l2(o, o_r) <= 5e-3 and O.rel_l2(ht, ht_r) <= 5e-3


def test_backward_raises():
    inp = make_inputs(34, 1, 4, 1, 64, 64)
    t = [x.float().to(DEV).requires_grad_() for x in (inp.q, inp.k, inp.v, inp.a, inp.b, inp.gk)]
    o, _ = fused_recurrent_dplr_delta_rule(*t, 2, scale=1.0)
    with pytest.raises(NotImplementedError):
        o.sum().backward()
