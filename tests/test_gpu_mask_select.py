"""Row-statistic mask methods on the GPU (top-k, statistical top-k, union over rows) and the sketch
threshold, against the oracle.  Top-k and the sketch threshold involve only comparisons, so they must
match bit for bit, ties included; the statistical cut is a floating-point sum, so mask bits are compared
outside a guard band around the cut that is much wider than the rounding difference (and asserted small)."""
import base64
import json
import os

import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _scores(seed, B, I, kind):
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((B, I)).astype(np.float32)
    if kind == "coarse":          # many equal scores: the k-th largest is shared by several indices
        s = (np.round(s * 4) / 4).astype(np.float32)
        s[s == 0] = np.where(rng.random((s == 0).sum()) < 0.5, np.float32(0.0), np.float32(-0.0))
    elif kind == "wide":          # exponents spread over many radix digits, both signs
        s = (s * np.exp(rng.uniform(-30, 30, size=s.shape))).astype(np.float32)
    elif kind == "constant":
        s[:] = np.float32(1.5)
    return s


@pytest.mark.parametrize("B,I,kind", [
    (1, 8192, "normal"), (1, 8192, "coarse"), (1, 14336, "wide"), (4, 11008, "normal"), (16, 14336, "coarse"),
    (8, 8192, "wide"), (3, 37, "coarse"), (2, 1000, "normal"), (1, 5, "normal"), (5, 1023, "constant"),
    (2, 40000, "coarse"),          # rows too long for the LDS copy: every pass reads the row again
])
def test_topk_bit_exact(B, I, kind):
    s = _scores(B * 31 + I, B, I, kind)
    sd = torch.from_numpy(s).to(DEV)
    ks = sorted({0, 1, 2, max(1, I // 7), max(1, int(I * 0.3)), I - 1, I, I + 5})
    for k in ks:
        want = oracle.mask_topk(s, k) if k > 0 else np.zeros(I, bool)
        got, cut = st.mask_select(sd, "topk", k=k, return_cutoff=True)
        got = got.cpu().numpy()
        assert np.array_equal(got, want), f"k={k}: {np.flatnonzero(got != want)[:8]}"
        if B == 1:
            assert got.sum() == min(k, I)
        if 0 < k < I:
            kth = -np.sort(-s, axis=1)[:, k - 1]
            assert np.array_equal(cut.cpu().numpy(), kth)


def test_topk_repeated_calls_share_workspace():
    """The ticket word that elects the block doing the union must be left ready for the next call."""
    for rep in range(4):
        B, I = (6, 3000) if rep % 2 == 0 else (16, 9000)
        s = _scores(100 + rep, B, I, "coarse")
        got = st.mask_select(torch.from_numpy(s).to(DEV), "topk", k=I // 5).cpu().numpy()
        assert np.array_equal(got, oracle.mask_topk(s, I // 5))


def test_topk_matches_torch_topk_scatter():
    """Without ties the result is what the reference's topk + scatter gives (src/modeling_skip.py:209-211)."""
    B, I, k = 4, 8192, 1024
    s = torch.randn(B, I, generator=torch.Generator().manual_seed(3))
    idx = s.topk(k, sorted=False)[1]
    want = torch.zeros(B, I, dtype=torch.bool).scatter_(-1, idx, True).any(0)
    assert torch.equal(st.mask_select(s.to(DEV), "topk", k=k).cpu(), want)


@pytest.mark.parametrize("B,I,kind,z", [
    (1, 8192, "normal", 0.5244), (1, 14336, "normal", -0.3), (4, 11008, "normal", 1.2816), (16, 8192, "normal", 0.0),
    (3, 37, "normal", 0.7), (2, 40000, "normal", 0.6745), (2, 512, "constant", 0.5),
])
def test_statistical_against_oracle(B, I, kind, z):
    s = _scores(B * 17 + I, B, I, kind)
    want, cut_ref = oracle.mask_statistical(s, z)
    got, cut = st.mask_select(torch.from_numpy(s).to(DEV), "statistical_topk", std_multiplier=z, return_cutoff=True)
    got, cut = got.cpu().numpy(), cut.cpu().numpy()
    scale = np.abs(s).max(1)
    assert (np.abs(cut - cut_ref) <= 1e-6 * scale).all()
    near = (np.abs(s - cut_ref[:, None]) <= 4e-6 * scale[:, None]).any(0)
    assert not ((got != want) & ~near).any()
    if kind != "constant":
        assert near.sum() <= 3
    # and against the reference's own formulation in torch (fp32 mean / std / compare)
    t = torch.from_numpy(s)
    m = (t > t.mean(-1, keepdim=True) + t.std(-1, keepdim=True, unbiased=False) * z).any(0).numpy()
    assert not ((got != m) & ~near).any()


def test_mask_select_errors():
    s = torch.zeros(2, 64, device=DEV)
    with pytest.raises(ValueError):
        st.mask_select(s, "median")
    with pytest.raises(ValueError):
        st.mask_select(s.half(), "topk", k=3)
    with pytest.raises(RuntimeError):
        st.mask_select(s.cpu(), "topk", k=3)


def test_projection_mask_methods():
    """FastLoRAProjection.mask with every method of SkipDecoderLayer._compute_binary_mask."""
    g = torch.Generator().manual_seed(8)
    B, H, r, I = 3, 512, 32, 2048
    A = (torch.randn(r, H, generator=g) * 0.05).half()
    Bm = (torch.randn(I, r, generator=g) * 0.05).half()
    x = torch.randn(B, H, generator=g).half()
    proj = st.FastLoRAProjection(A.to(DEV), Bm.to(DEV))
    s_dev = proj(x.to(DEV))
    s = s_dev.cpu().numpy()
    k = int(H * (1 - 0.7))     # the reference sizes k from hidden_size (src/modeling_skip.py:135,144)
    assert np.array_equal(proj.mask(x.to(DEV), "topk", k=k).cpu().numpy(), oracle.mask_topk(s, k))
    z = 0.5244
    want, cut = oracle.mask_statistical(s, z)
    got = proj.mask(x.to(DEV), "statistical_topk", std_multiplier=z).cpu().numpy()
    near = (np.abs(s - cut[:, None]) <= 4e-6 * np.abs(s).max()).any(0)
    assert not ((got != want) & ~near).any()


# ------------------------------------------------------------------ sketch threshold
def _b64_f32(t):
    return np.frombuffer(base64.b64decode(t), dtype="<f4").copy()


def test_approx_topk_reference_vectors():
    with open(os.path.join(os.path.dirname(__file__), "golden", "approx_topk.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        sc = _b64_f32(c["scores_f32_b64"]).reshape(c["B"], c["F"])
        want = _b64_f32(c["threshold_f32_b64"])
        got = st.approx_topk_threshold(torch.from_numpy(sc).to(DEV), c["k"])
        assert tuple(got.shape) == (c["B"], 1)
        assert np.array_equal(got.cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32)), (c["F"], c["k"])


@pytest.mark.parametrize("B,F,kind", [(1, 8192, "normal"), (4, 14336, "coarse"), (16, 11008, "wide"), (3, 4097, "normal"),
                                      (2, 7, "normal"), (1, 4, "coarse"), (2, 100000, "normal")])
def test_approx_topk_bit_exact(B, F, kind):
    s = _scores(F + B, B, F, kind)
    sd = torch.from_numpy(s).to(DEV)
    for k in sorted({1, max(1, F // 10), max(1, F // 2), F}):
        want = oracle.approx_topk_threshold(s, k)
        got = st.approx_topk_threshold(sd, k).cpu().numpy().reshape(-1)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), k


def test_approx_topk_f64_reference_vectors_and_oracle():
    """Double scores (the reference dispatches on the type, approx_topk.h:33): bit-equal to the vectors written from
    the compiled reference and to the oracle, incl. values whose bit patterns agree in their upper halves."""
    import base64
    with open(os.path.join(os.path.dirname(__file__), "golden", "approx_topk_f64.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        sc = np.frombuffer(base64.b64decode(c["scores_f64_b64"]), dtype="<f8").copy().reshape(c["B"], c["F"])
        want = np.frombuffer(base64.b64decode(c["threshold_f64_b64"]), dtype="<f8")
        got = st.approx_topk_threshold(torch.from_numpy(sc).to(DEV), c["k"])
        assert got.dtype == torch.float64 and tuple(got.shape) == (c["B"], 1)
        assert np.array_equal(got.cpu().numpy().reshape(-1), want), (c["B"], c["F"], c["k"])
    rng = np.random.default_rng(8)
    for F in (4, 100, 4096, 14336):
        for kind in ("normal", "close", "ties"):
            s = rng.standard_normal((3, F))
            if kind == "close":
                s = -3.0 + s * 1e-13
            elif kind == "ties":
                s = np.round(s * 2) / 2
            for k in sorted({1, max(1, F // 9), F}):
                want = oracle.approx_topk_threshold(s, k)
                got = st.approx_topk_threshold(torch.from_numpy(s).to(DEV), k).cpu().numpy().reshape(-1)
                assert np.array_equal(got, want), (F, kind, k)


def test_approx_topk_errors():
    s = torch.zeros(2, 64, device=DEV)
    for bad in (lambda: st.approx_topk_threshold(s, 0), lambda: st.approx_topk_threshold(s, 65),
                lambda: st.approx_topk_threshold(s[0], 3)):
        with pytest.raises(RuntimeError):
            bad()
