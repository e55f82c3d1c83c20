"""Pins of oracle/layer_oracle.py (CPU, float64) and host-side checks of hdla_hip.layer that need no GPU."""
import pytest
import torch
import torch.nn.functional as F

from hdla_hip.layer import HDLA_Custom, RecurrentCache, get_activation_fn
from oracle import hrdplr_oracle as O
from oracle import layer_oracle as LO
from oracle import normalize_oracle as NO


def _sd(seed, d, H, beta=True, gate=True, std=0.5):
    g = torch.Generator().manual_seed(seed)
    D = d // H
    r = lambda *s: std * torch.randn(*s, generator=g, dtype=torch.float64) / s[-1] ** 0.5 * 4
    sd = {"q_proj.weight": r(d, d), "k_proj.weight": r(d, d), "v_proj.weight": r(d, d), "f_proj.0.weight": r(D, d),
          "f_proj.1.weight": r(d, D), "o_proj.weight": r(d, d), "norm.weight": 1 + 0.1 * r(d)}
    if beta:
        sd["bet_proj.weight"] = r(H, d)
    if gate:
        sd["output_gate.0.weight"] = r(D, d)
        sd["output_gate.1.weight"] = r(d, D)
    return sd


def _x(seed, *s):
    return torch.randn(*s, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_single_head_reduces_to_the_written_out_recurrence():
    d, n = 16, 9
    sd, x = _sd(0, d, 1), _x(1, 1, n, d)
    out, S = LO.hdla_layer(sd, x, 1)
    q = F.silu(x[0] @ sd["q_proj.weight"].T)
    k = F.silu(x[0] @ sd["k_proj.weight"].T)
    v = F.silu(x[0] @ sd["v_proj.weight"].T)
    f = torch.sigmoid(x[0] @ sd["f_proj.0.weight"].T @ sd["f_proj.1.weight"].T)
    beta = 2 * torch.sigmoid(x[0] @ sd["bet_proj.weight"].T)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + d * 1e-5)
    St, I, rows = torch.zeros(d, d, dtype=torch.float64), torch.eye(d, dtype=torch.float64), []
    for t in range(n):
        P = I - beta[t] * torch.outer(k[t], k[t])
        St = P @ torch.diag(f[t]) @ P @ St + torch.outer(k[t], v[t])           # hdla_custom.py:46-48,270-272
        rows.append(St.T @ q[t])
    o = torch.stack(rows)
    gate = torch.sigmoid(x[0] @ sd["output_gate.0.weight"].T @ sd["output_gate.1.weight"].T)
    og = o * gate
    o = og / torch.sqrt((og * og).mean(-1, keepdim=True) + 1e-5) * sd["norm.weight"]
    assert torch.allclose(out[0], o @ sd["o_proj.weight"].T, rtol=1e-10, atol=1e-10)
    assert torch.allclose(S[0, 0], St, rtol=1e-10, atol=1e-10)


def test_causal_and_state_hand_over():
    d, H, n = 32, 4, 12
    sd, x = _sd(2, d, H), _x(3, 2, n, d)
    full, S = LO.hdla_layer(sd, x, H)
    pre, S1 = LO.hdla_layer(sd, x[:, :7], H)
    assert torch.allclose(full[:, :7], pre, rtol=1e-12, atol=1e-12)            # later tokens do not reach back
    rest, S2 = LO.hdla_layer(sd, x[:, 7:], H, initial_state=S1)
    assert torch.allclose(full[:, 7:], rest, rtol=1e-10, atol=1e-10)
    assert torch.allclose(S, S2, rtol=1e-10, atol=1e-10)


def test_blocks_split_key_channels_and_share_values():
    d, H, n, nb = 32, 2, 6, 2
    sd, x = _sd(4, d, H), _x(5, 1, n, d)
    out, S = LO.hdla_layer(sd, x, H, num_blocks=nb)
    assert S.shape == (1, H * nb, d // H // nb, d // H)
    # block j of head h sees key channels [j*8, (j+1)*8) of that head and all of its value channels: a layer whose
    # q/k/f projections keep only those channels (one block, other channels' rows zero) gives that block's share
    o_pre = []
    for j in range(nb):
        keep = torch.zeros(d, dtype=torch.bool)
        for h in range(H):
            keep[h * 16 + j * 8: h * 16 + (j + 1) * 8] = True
        # share of block j before the norm = recurrence on its channels only
        q = F.silu(x @ sd["q_proj.weight"].T)[..., keep].reshape(1, n, H, 8)
        k = NO.l2_norm(F.silu(x @ sd["k_proj.weight"].T)[..., keep].reshape(1, n, H, 8))
        lf = F.logsigmoid(x @ sd["f_proj.0.weight"].T @ sd["f_proj.1.weight"].T)[..., keep].reshape(1, n, H, 8)
        v = F.silu(x @ sd["v_proj.weight"].T).reshape(1, n, H, 16)
        beta = 2 * torch.sigmoid(x @ sd["bet_proj.weight"].T).unsqueeze(-1)
        a, b = O.parameterize_a_b(beta, k, lf)
        o, _ = O.recurrence(q, k, v, a, b, lf, 1.0, None)
        o_pre.append(o)
    o = (o_pre[0] + o_pre[1]).reshape(1, n, d)
    gate = x @ sd["output_gate.0.weight"].T @ sd["output_gate.1.weight"].T
    ref = NO.rms_norm_fused_gate(o, gate, sd["norm.weight"]) @ sd["o_proj.weight"].T
    assert torch.allclose(out, ref, rtol=1e-10, atol=1e-10)


def test_masked_tokens_leave_the_state_alone():
    d, H, n = 32, 4, 8
    sd, x = _sd(6, d, H), _x(7, 1, n, d)
    mask = torch.ones(1, n, dtype=torch.long)
    mask[0, :3] = 0                                                            # left padding
    _, S = LO.hdla_layer(sd, x, H, attention_mask=mask)
    _, S_ref = LO.hdla_layer(sd, x[:, 3:], H)
    assert torch.allclose(S, S_ref, rtol=1e-10, atol=1e-10)                    # k = 0, log_f = 0: identity step


def test_module_has_the_reference_parameter_names_and_init():
    m = HDLA_Custom(64, 4, use_offset=True)
    assert set(m.state_dict()) == {"q_proj.weight", "k_proj.weight", "v_proj.weight", "f_proj.0.weight",
                                   "f_proj.1.weight", "bet_proj.weight", "o_proj.weight", "norm.weight",
                                   "output_gate.0.weight", "output_gate.1.weight", "offset"}
    assert float(m.o_proj.weight.detach().abs().max()) == 0.0                           # rescale_type 2 (the default)
    assert torch.allclose(torch.sigmoid(m.offset), torch.full((64,), 0.99))
    bound = 0.01 * (6 / 128) ** 0.5                                            # xavier_uniform with gain 0.01
    assert float(m.q_proj.weight.detach().abs().max()) <= bound
    m1 = HDLA_Custom(64, 4, rescale_type=1, num_hidden_layers=8, token_mixer_init_type=2, use_beta=False,
                     use_output_gate=False)
    assert "bet_proj.weight" not in m1.state_dict() and "output_gate.0.weight" not in m1.state_dict()
    assert float(m1.o_proj.weight.detach().abs().max()) <= 2 ** -0.5 * (6 / 128) ** 0.5 / 4 + 1e-9
    with pytest.raises(AssertionError):
        HDLA_Custom(64, 4, causal=False)
    assert get_activation_fn("relu2")(torch.tensor([-1.0, 3.0])).tolist() == [0.0, 9.0]
    assert get_activation_fn("none")(torch.tensor([2.0])).item() == 2.0


def test_recurrent_cache_contract():
    c = RecurrentCache()
    assert len(c) == 0 and c.get_seq_length(0) == 0
    c.update(recurrent_state=["S0"], layer_idx=0, offset=5)
    c.update(recurrent_state=["S1"], layer_idx=1, offset=5)
    c.update(recurrent_state=["S0b"], layer_idx=0, offset=1)
    assert len(c) == 2 and c[0]["recurrent_state"][0] == "S0b" and c.get_seq_length(0) == 6 and c.get_seq_length(1) == 5


def test_gathered_projection_weight_is_cached_only_in_evaluation_mode_without_gradients():
    m = HDLA_Custom(64, 4)
    heads = [m.q_proj, m.k_proj, m.v_proj, m.bet_proj, m.f_proj[0], m.output_gate[0]]
    w1, _ = m._gathered(heads)
    assert w1.requires_grad and w1.shape == (3 * 64 + 4 + 16 + 16, 64)          # part of the graph: rebuilt per call
    assert m._gathered(heads)[0] is not w1
    with torch.no_grad():
        assert m._gathered(heads)[0] is not m._gathered(heads)[0]                # training mode: never cached
        m.eval()
        a, _ = m._gathered(heads)
        assert m._gathered(heads)[0] is a and not a.requires_grad                # reused
        m.k_proj.weight.mul_(2.0)                                                # a parameter changes in place
        b, _ = m._gathered(heads)
        assert b is not a and torch.equal(b[64:128], m.k_proj.weight)
        m.k_proj.weight.data.mul_(0.5)                                           # untracked write: needs reset_cache()
        assert m._gathered(heads)[0] is b
        m.reset_cache()
        c, _ = m._gathered(heads)
        assert c is not b and torch.equal(c[64:128], m.k_proj.weight)
        m.train()
        m.eval()                                                                 # mode switches drop it too
        assert m._gathered(heads)[0] is not c
        d = m._gathered(heads)[0]
        m.load_state_dict({k: v.clone() for k, v in m.state_dict().items()})
        assert m._gathered(heads)[0] is not d
    m.requires_grad_(False)
    e = m._gathered(heads)[0]
    assert m._gathered(heads)[0] is e                                            # frozen parameters: cached with grad mode on
    m2 = m.to(torch.bfloat16)
    assert m2._gathered(heads)[0].dtype == torch.bfloat16                        # new storage, new entry


def test_golden_fixture_layer0():
    """Seeded fixture of the normalisation and layer oracles (tests/golden/layer0.npz, written by
    tests/golden/make_golden.py from this repository's own float64 code): guards the oracles against drift."""
    import os
    import sys
    import numpy as np
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
    from make_golden import layer_case
    sd, x, gate, H = layer_case()
    fix = np.load(os.path.join(os.path.dirname(__file__), "golden", "layer0.npz"))
    out, S = LO.hdla_layer(sd, x, H)
    close = lambda a, name: np.testing.assert_allclose(a.numpy(), fix[name], rtol=1e-12, atol=1e-12)
    close(out, "layer_out")
    close(S, "layer_state")
    close(NO.rms_norm_fused_gate(x, gate, sd["norm.weight"], eps=1e-5), "rms_gate_pre")
    close(NO.normalize(x, sd["norm.weight"], gate, "sigmoid", "post", c=8 ** 0.5, eps=1e-3, num_groups=4), "group_post")
    close(NO.l2_norm(x.reshape(2, 10, 4, 8)), "l2")
