"""Committed fixtures under tests/golden/: the known answers the reference's own tests hold
(reference_known_answers.json) and seeded vectors written by tests/golden/make_vectors.py
(seeded_vectors.npz).  CPU tests check both oracles against them; GPU tests check the HIP path."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ["small_tail", "temp_bias_ignore", "two_tiles"]


@pytest.fixture(scope="module")
def known():
    with open(os.path.join(GOLDEN, "reference_known_answers.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLDEN, "seeded_vectors.npz"))


def _case(vec, name):
    get = lambda k: vec[f"{name}/{k}"] if f"{name}/{k}" in vec.files else None
    ign = -100 if bool((vec[f"{name}/targets"] == -100).any()) else None
    return {k: get(k) for k in ("hidden", "weight", "bias", "targets", "grad", "logp", "lse", "dh",
                                "dw", "db")}, float(vec[f"{name}/temperature"]), ign


def _rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


# ------------------------------------------------------------------ CPU: oracles vs fixtures
def test_oracles_reproduce_reference_known_answers(known, c_oracle):
    for k in known["logp_from_logits"]:
        logits = torch.tensor(k["logits"])
        ids = torch.tensor(k["ids"])
        got = O.linear_logp(logits, torch.eye(logits.shape[1]), ids, temperature=k["temperature"])
        assert np.allclose(got.numpy(), k["expected"], atol=1e-6), k["source"]
        got_c, _ = c_oracle.linear_logp(logits.numpy(), np.eye(logits.shape[1]), k["ids"],
                                        temperature=k["temperature"])
        assert np.allclose(got_c, k["expected"], atol=1e-12), k["source"]
        if k["temperature"] == 1.0:
            assert np.allclose(O.logp_from_logits(logits, ids).numpy(), k["expected"], atol=1e-6)
    for k in known["masked_mean"]:
        got = O.masked_mean(torch.tensor(k["values"]), torch.tensor(k["mask"], dtype=torch.bool))
        assert got.item() == pytest.approx(k["expected"], abs=1e-6), k["source"]
    for k in known["ratio_kl"]:
        cur = torch.tensor(k["current"])
        mask = torch.tensor(k["mask"], dtype=torch.bool)
        r = O.policy_ratio(cur, cur + k["old_offset"], mask)
        kl = O.reference_kl(cur, cur + k["ref_offset"], mask)
        assert np.allclose(r[mask].numpy(), k["expected_ratio_active"], atol=1e-6)
        assert np.allclose(kl[mask].numpy(), k["expected_kl_active"], atol=1e-7)
        assert torch.all(r[~mask] == k["expected_masked"]) and torch.all(kl[~mask] == 0.0)
    for k in known["group_advantages"]:
        got = O.group_advantages(torch.tensor(k["rewards"]), group_boundaries=k["group_boundaries"])
        assert np.allclose(got.numpy(), k["expected"], atol=1e-5), k["source"]
        got_c = c_oracle.group_advantages(np.array(k["rewards"]), k["group_boundaries"])
        assert np.allclose(got_c, k["expected"], atol=1e-9)


@pytest.mark.parametrize("name", CASES)
def test_torch_oracle_reproduces_seeded_vectors(vec, name):
    c, temp, ign = _case(vec, name)
    t = lambda x: None if x is None else torch.from_numpy(np.asarray(x))
    logp, lse = O.linear_logp(t(c["hidden"]), t(c["weight"]), t(c["targets"]), t(c["bias"]),
                              temperature=temp, ignore_index=ign, return_lse=True)
    assert np.abs(logp.numpy() - c["logp"]).max() < 1e-5
    live = c["targets"] != -100
    assert np.abs(lse.numpy() - c["lse"])[live].max() < 1e-5
    assert np.all(logp.numpy()[~live] == 0.0)
    dh, dw, db = O.linear_logp_backward(t(c["grad"]), t(c["hidden"]), t(c["weight"]),
                                        t(c["targets"]), t(c["bias"]), temperature=temp,
                                        ignore_index=ign)
    assert _rel(dh.numpy(), c["dh"]) < 1e-5 and _rel(dw.numpy(), c["dw"]) < 1e-5
    if c["db"] is not None:
        assert _rel(db.numpy(), c["db"]) < 1e-5


def test_c_oracle_reproduces_seeded_vectors(vec, c_oracle):
    for name in CASES:
        c, temp, ign = _case(vec, name)
        logp, lse = c_oracle.linear_logp(c["hidden"], c["weight"], c["targets"], c["bias"],
                                         temperature=temp, ignore_index=ign)
        assert np.array_equal(logp, c["logp"]) and np.array_equal(lse, c["lse"])
    out3, dcur = c_oracle.grpo_from_logp(vec["grpo/cur"], vec["grpo/old"], vec["grpo/ref"],
                                         np.repeat(vec["grpo/adv"][:, None], 17, axis=1),
                                         vec["grpo/mask"], clip_eps=0.2, beta=0.04)
    assert np.array_equal(out3, vec["grpo/out3"])
    t = torch.from_numpy
    loss, pol, kl, grad = O.grpo_loss_from_logp(t(vec["grpo/cur"]), t(vec["grpo/old"]),
                                                t(vec["grpo/ref"]), t(vec["grpo/adv"]).float(),
                                                t(vec["grpo/mask"]), clip_eps=0.2, beta=0.04)
    assert np.allclose([loss.item(), pol.item(), kl.item()], vec["grpo/out3"], atol=1e-6)
    assert np.allclose(grad.numpy(), vec["grpo/dcur"], atol=1e-7)


# ------------------------------------------------------------------ GPU: HIP path vs fixtures
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,atol,gtol", [(torch.bfloat16, 1e-3, 2e-2), (torch.float16, 1e-3, 2e-2),
                                             (torch.float32, 1e-5, 1e-4)])
@pytest.mark.parametrize("name", CASES)
def test_hip_path_matches_seeded_vectors(vec, name, dtype, atol, gtol):
    from rl_kernel_amd.ops import linear_logp as LL

    dev = torch.device("cuda:0")
    c, temp, ign = _case(vec, name)
    d = lambda x, dt=None: None if x is None else torch.from_numpy(np.asarray(x)).to(dev, dt)
    hidden, weight = d(c["hidden"], dtype), d(c["weight"], dtype)   # bf16-exact inputs
    bias = d(c["bias"], torch.float32)
    targets = d(c["targets"])
    logp, lse, err = LL.fused_linear_logp_forward(hidden, weight, targets, bias, temperature=temp,
                                                  ignore_index=ign)
    assert int(err.item()) == 0
    live = c["targets"] != -100
    assert np.abs(logp.cpu().numpy() - c["logp"]).max() < atol
    assert np.abs(lse.cpu().numpy() - c["lse"])[live].max() < atol
    assert np.all(logp.cpu().numpy()[~live] == 0.0)                 # exact zeros on ignored rows
    dh, dw, db = LL.fused_linear_logp_backward(d(c["grad"]), hidden, weight, targets, lse, bias,
                                               temperature=temp, ignore_index=ign)
    assert _rel(dh.float().cpu().numpy(), c["dh"]) < gtol
    assert _rel(dw.float().cpu().numpy(), c["dw"]) < gtol
    if c["db"] is not None:
        assert _rel(db.float().cpu().numpy(), c["db"]) < gtol
    assert np.all(dh.float().cpu().numpy()[~live] == 0.0)


@pytest.mark.gpu
def test_hip_epilogue_matches_known_answers_and_seeded_vectors(known, vec):
    from rl_kernel_amd.ops import grpo as GR
    from rl_kernel_amd.ops.logp import logp_from_logits

    dev = torch.device("cuda:0")
    for k in known["logp_from_logits"]:
        if k["temperature"] != 1.0:
            continue
        logits = torch.tensor(k["logits"], device=dev)
        got = logp_from_logits(logits, torch.tensor(k["ids"], device=dev),
                               torch.empty(logits.shape[0], device=dev))
        assert np.allclose(got.float().cpu().numpy(), k["expected"], atol=1e-6), k["source"]
    for k in known["group_advantages"]:
        got = GR.group_advantages(torch.tensor(k["rewards"], device=dev),
                                  group_boundaries=k["group_boundaries"])
        assert np.allclose(got.cpu().numpy(), k["expected"], atol=1e-5), k["source"]
    for k in known["ratio_kl"]:
        cur = torch.tensor(k["current"], device=dev)
        mask = torch.tensor(k["mask"], dtype=torch.bool, device=dev)
        zeros = torch.zeros_like(cur)
        _, ratio, kl, _, _ = GR.grpo_from_logp_raw(cur, cur + k["old_offset"], cur + k["ref_offset"],
                                                   zeros, mask, clip_eps=0.2, beta=0.0,
                                                   want_grad=False, want_terms=True)
        assert np.allclose(ratio[mask].cpu().numpy(), k["expected_ratio_active"], atol=1e-6)
        assert np.allclose(kl[mask].cpu().numpy(), k["expected_kl_active"], atol=1e-7)
        assert torch.all(ratio[~mask] == 0.0) and torch.all(kl[~mask] == 0.0)
    t = lambda x: torch.from_numpy(np.asarray(x)).to(dev)
    adv = GR.group_advantages(t(vec["grpo/rewards"]), samples_per_prompt=3)
    assert np.allclose(adv.cpu().numpy(), vec["grpo/adv"], atol=1e-5)
    out3, _, _, dcur, _ = GR.grpo_from_logp_raw(t(vec["grpo/cur"]), t(vec["grpo/old"]),
                                                t(vec["grpo/ref"]), t(vec["grpo/adv"]).float(),
                                                t(vec["grpo/mask"]), clip_eps=0.2, beta=0.04,
                                                want_grad=True)
    assert np.allclose(out3.cpu().numpy(), vec["grpo/out3"], atol=1e-6)
    assert np.allclose(dcur.cpu().numpy(), vec["grpo/dcur"], atol=1e-7)
