"""LoRA predictor + threshold mask + batch union on the GPU vs the oracle.  Scores are floating point
(tolerance); masks are bits and must be exact, so thresholds are placed in a gap between scores that is
much wider than the rounding difference between the two implementations (the guard band is asserted)."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd import synthetic as syn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _weights(seed, B, H, r, I, dtype):
    g = torch.Generator().manual_seed(seed)
    tdt = getattr(torch, dtype)
    A = (torch.randn(r, H, generator=g) * 0.02).to(tdt)
    Bm = (torch.randn(I, r, generator=g) * 0.02).to(tdt)
    x = torch.randn(B, H, generator=g).to(tdt)
    return x, A, Bm


@pytest.mark.parametrize("B,H,r,I,dtype,frac", [
    (1, 2048, 64, 8192, "float32", 0.30),      # Llama-3.2-1B layer, fp32
    (1, 3072, 128, 8192, "float16", 0.35),     # Llama-3.2-3B layer, fp16
    (8, 4096, 256, 14336, "bfloat16", 0.25),   # Mistral-7B layer, bf16, batch union
    (1, 4096, 440, 11008, "float16", 0.10),    # ReLU-Llama-7B layer: rank int(0.04 * I), 55 chunks per row
    (16, 3072, 128, 8192, "bfloat16", 0.30),   # Llama-3.2-3B layer, bf16, decode batch 16
    (3, 128, 8, 50, "float16", 0.5),           # tiny / ragged
    (2, 64, 4, 17, "float32", 0.5),
    (1, 1024, 1024, 300, "float16", 0.4),      # rank rows longer than one pass of the wave
    (150, 1024, 64, 2048, "float16", 0.02),    # more rows than one pass takes (64): three passes, mask bytes accumulate
    (70, 512, 256, 1024, "bfloat16", 0.02),    # rank 256: a pass takes 56 rows
])
def test_scores_and_mask(B, H, r, I, dtype, frac):
    x, A, Bm = _weights(B * 7 + r, B, H, r, I, dtype)
    s_ref = oracle.predictor_scores(x.float().numpy(), A.float().numpy(), Bm.float().numpy())
    m, s = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), 0.0, True, return_scores=True)
    s = s.cpu().numpy()
    scale = np.abs(s_ref).max()
    assert np.abs(s - s_ref).max() <= 2e-6 * scale + 1e-9           # fp32 accumulation on both sides
    guard = 8e-6 * scale
    thr = syn.threshold_for_fraction(s_ref.max(0) if B > 1 else s_ref, frac, guard=0.0)
    near = np.abs(s_ref - thr) < guard
    for ge in (True, False):
        want = oracle.mask_threshold(s_ref, thr, ge)
        got = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), thr, ge).cpu().numpy()
        diff = got != want
        assert not (diff & ~near.any(0)).any(), "mask bit differs outside the guard band"
        assert diff.sum() <= near.any(0).sum()
    assert near.sum() <= 3, f"guard band population {near.sum()}"      # expected 0, reported if not


def test_naive_threshold_is_score_ge_zero():
    x, A, Bm = _weights(1, 2, 256, 16, 512, "float32")
    # make some scores exactly zero: a zero row of Bm gives score 0 for every input row
    Bm[5] = 0.0
    Bm[77] = 0.0
    m_ge = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), 0.0, True).cpu().numpy()
    m_gt = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), 0.0, False).cpu().numpy()
    assert m_ge[5] and m_ge[77] and not m_gt[5] and not m_gt[77]     # >= vs > on an exact tie
    s = oracle.predictor_scores(x.numpy(), A.numpy(), Bm.numpy())
    safe = np.abs(s).min(0) > 1e-6
    assert np.array_equal(m_ge[safe], (s >= 0).any(0)[safe])


@pytest.mark.parametrize("method", ["naive", "topk", "statistical_topk"])
def test_mask_methods_of_the_reference(method):
    """The three sparsity methods of SkipDecoderLayer._compute_binary_mask, union over rows included."""
    B, H, r, I = 4, 512, 32, 2048
    x, A, Bm = _weights(3, B, H, r, I, "float32")
    pred = st.FastLoRAProjection(A.to(DEV), Bm.to(DEV))
    s_ref = oracle.predictor_scores(x.numpy(), A.numpy(), Bm.numpy())
    if method == "naive":
        got = pred.mask(x.to(DEV), "naive").cpu().numpy()
        want, margin = oracle.mask_threshold(s_ref, 0.0, True), np.abs(s_ref).min(0)
    elif method == "topk":
        k = 300
        got = pred.mask(x.to(DEV), "topk", k=k).cpu().numpy()
        want = oracle.mask_topk(s_ref, k)
        kth = np.sort(s_ref, axis=1)[:, -k][:, None]
        margin = np.abs(s_ref - kth).min(0)
    else:
        z = float(torch.distributions.normal.Normal(0, 1).icdf(torch.tensor(0.7)))
        got = pred.mask(x.to(DEV), "statistical_topk", std_multiplier=z).cpu().numpy()
        want, cut = oracle.mask_statistical(s_ref, z)
        margin = np.abs(s_ref - cut[:, None]).min(0)
    safe = margin > 1e-5 * np.abs(s_ref).max()
    assert safe.mean() > 0.99
    assert np.array_equal(got[safe], want[safe])


def test_predictor_argument_errors():
    x, A, Bm = _weights(0, 1, 64, 8, 32, "float32")
    with pytest.raises(ValueError):
        st.predictor_mask(x.to(DEV), A.to(DEV)[:, :32], Bm.to(DEV))
    with pytest.raises(TypeError):
        st.predictor_mask(x.to(DEV), A.to(DEV).half(), Bm.to(DEV))
    with pytest.raises(ValueError):
        st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), out=torch.zeros(31, dtype=torch.bool, device=DEV))
    sd = {"down.weight": A, "up.weight": Bm}
    p = st.FastLoRAProjection.from_state_dict(sd, device=DEV, dtype=torch.float32)   # the reference's checkpoint keys
    assert p.lora_size == 8 and p.intermediate_size == 32


def test_loaded_checkpoints_drive_the_hip_predictor(tmp_path):
    """Predictor files as the reference's trainer writes them (fp32 state dicts with keys down.weight [r,H] and
    up.weight [I,r] under final_predictor_layer_{i}_lora_{pct}pct.pt, src/trainer.py:569-585), loaded the way
    benchmark.py:460-468 consumes them, here onto the GPU in fp16: the loaded predictors' scores and masks against
    the oracle on the same (fp16-rounded) weights."""
    H, I = 3072, 8192
    r = int(I * 0.016)          # the trainer's sizing rule int(I * pct / 100) at 1.6 % -> 131 -> not a multiple of 8
    r = (r // 8) * 8            # 128: rank rows must be 16-byte multiples in fp16
    g = torch.Generator().manual_seed(21)
    want = []
    for layer in range(2):
        sd = {"down.weight": torch.randn(r, H, generator=g) * 0.02, "up.weight": torch.randn(I, r, generator=g) * 0.02}
        torch.save(sd, tmp_path / st.FastLoRAProjection.checkpoint_name(layer, 1.6))
        want.append(sd)
    preds = st.load_predictors(str(tmp_path), 2, 1.6, device=DEV, dtype=torch.float16)
    x = torch.randn(2, H, generator=g).half()
    for p, sd in zip(preds, want):
        assert p.down_weight.is_cuda and p.down_weight.dtype == torch.float16 and p.lora_size == r
        A, Bm = sd["down.weight"].half().float().numpy(), sd["up.weight"].half().float().numpy()
        s_ref = oracle.predictor_scores(x.float().numpy(), A, Bm)
        s = p(x.to(DEV)).cpu().numpy()
        scale = np.abs(s_ref).max()
        assert np.abs(s - s_ref).max() <= 2e-6 * scale
        thr = syn.threshold_for_fraction(s_ref.max(0), 0.35)
        near = (np.abs(s_ref - thr) < 8e-6 * scale).any(0)
        got = p.mask(x.to(DEV), "threshold", thr=thr).cpu().numpy()
        assert np.array_equal(got[~near], oracle.mask_threshold(s_ref, thr, True)[~near]) and near.sum() <= 3
        got_naive = p.mask(x.to(DEV), "naive").cpu().numpy()
        safe = np.abs(s_ref).min(0) > 8e-6 * scale
        assert np.array_equal(got_naive[safe], oracle.mask_threshold(s_ref, 0.0, True)[safe]) and safe.mean() > 0.999


@pytest.mark.parametrize("dtype,B,H,r,I", [("float16", 1, 3072, 128, 8192), ("bfloat16", 4, 4096, 256, 14336)])
def test_scores_rounded_to_the_storage_type(dtype, B, H, r, I):
    """round_to_storage: the rank-r intermediate and the scores as two half-precision modules hand them on
    (FastLoRAProjection in an fp16 / bf16 model, src/modeling_skip.py:52-53) against the oracle's restatement of that;
    and how many mask bits that moves against the fp32 scores at the benchmark's active fraction."""
    x, A, Bm = _weights(5, B, H, r, I, dtype)
    xs, As, Bs = x.float().numpy(), A.float().numpy(), Bm.float().numpy()
    want = oracle.predictor_scores(xs, As, Bs, storage=dtype)
    got = st.predictor_scores(x.to(DEV), A.to(DEV), Bm.to(DEV), round_to_storage=True).cpu().numpy()
    # every score is a value of the storage type
    tdt = getattr(torch, dtype)
    assert np.array_equal(torch.from_numpy(got).to(tdt).float().numpy(), got)
    # equal to the oracle's except where an fp32 sum sat within rounding distance of a tie between two storage values:
    # a score is then one step of the storage type off, or -- when it was an entry of the intermediate -- a few
    ulp = np.abs(want) * (2.0 ** -10 if dtype == "float16" else 2.0 ** -7) + 1e-30
    diff = np.abs(got - want)
    assert (diff <= 8 * ulp + 1e-3 * np.abs(want).max()).all() and (diff > 0).mean() < 0.02, \
        ((diff > 0).mean(), (diff / ulp).max())
    # masks: exact wherever the two implementations' scores agree; and the count of bits the rounding itself moves
    s32 = oracle.predictor_scores(xs, As, Bs)
    thr = syn.threshold_for_fraction(s32.max(0), 0.35)
    m_round = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), thr, True, round_to_storage=True).cpu().numpy()
    agree = (diff == 0).all(0)
    assert np.array_equal(m_round[agree], oracle.mask_threshold(want, thr, True)[agree])
    m_fp32 = st.predictor_mask(x.to(DEV), A.to(DEV), Bm.to(DEV), thr, True).cpu().numpy()
    moved = int((m_round != m_fp32).sum())
    print(f"{dtype}: {moved} of {I} mask bits differ between scores kept in fp32 and scores rounded to {dtype}")
    assert moved <= (40 if dtype == "float16" else 300)
    # fp32 storage: the flag changes nothing
    x32, A32, B32 = _weights(6, 1, 256, 16, 512, "float32")
    a = st.predictor_scores(x32.to(DEV), A32.to(DEV), B32.to(DEV), round_to_storage=True)
    b = st.predictor_scores(x32.to(DEV), A32.to(DEV), B32.to(DEV))
    assert torch.equal(a, b)
