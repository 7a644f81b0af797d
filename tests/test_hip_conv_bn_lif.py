"""Fused kernel-size-1 convolution / batch norm / LIF kernels against the float64 oracle
(``oracle/conv_bn_lif_oracle.py``, pinned on the CPU against torch's ``nn.Conv1d`` / ``nn.BatchNorm1d`` and this
package's torch-backend block).

Bars.  GEMMs with three bf16 terms per fp32 operand: 2e-6 of the row's sum of |products| (an fp32 GEMM's own bound is
K * 6e-8 of it); exact on operands whose products and sums fp32 holds exactly.  Batch norm + LIF: spikes identical
wherever the oracle's membrane potential is further than 1e-5 from the threshold (the test inputs are checked to hold
no closer neuron, so all spikes are compared), running statistics and gradients within 1e-5 relative of float64.
"""

import pytest
import torch
import torch.nn as nn

from oracle import conv_bn_lif_oracle as co
from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, layer, neuron, surrogate

from helpers import seeded_randn

pytestmark = pytest.mark.gpu

MARGIN = 1e-5


@pytest.fixture(scope="module")
def C():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import conv_bn_lif, library

    library.load()
    return conv_bn_lif


# ------------------------------------------------------------------------------------------------
# the three GEMMs
# ------------------------------------------------------------------------------------------------
# (token counts that are a multiple of 4 leave through the 16-byte epilogue, the others, which must be even, element by element)
SHAPES = [(3, 100, 50, 12), (2, 128, 32, 128), (5, 384, 384, 196), (1, 7, 3, 4), (4, 130, 257, 36), (16, 1152, 384, 196),
          (3, 70, 33, 6), (5, 200, 64, 198)]


@pytest.mark.parametrize("S,M,Kd,Lp", SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
def test_gemm_with_three_terms_has_fp32_accuracy(C, S, M, Kd, Lp, transpose):
    w = seeded_randn((Kd, M) if transpose else (M, Kd), 11, 0.0, 1.0)
    x = seeded_randn((S, Kd, Lp), 12, 0.1, 1.0)
    planes = C.split_weight(w.cuda(), transpose)
    got = C.pw_gemm(planes, 3, M, Kd, x.cuda(), 3).cpu().double()
    a = (w.t() if transpose else w).double()
    want = torch.einsum("mk,skl->sml", a, x.double())
    bound = torch.einsum("mk,skl->sml", a.abs(), x.double().abs())
    assert float(((got - want).abs() / bound).max()) < 2e-6
    # and better than what two terms give
    err3 = float((got - want).abs().max())
    got2 = C.pw_gemm(planes, 2, M, Kd, x.cuda(), 2).cpu().double()
    assert float(((got2 - want).abs() / bound).max()) < 3e-5
    assert err3 <= float((got2 - want).abs().max())


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (4, 384, 384, 196)])
def test_gemm_is_exact_on_spikes_times_dyadic_weights(C, S, M, Kd, Lp):
    g = torch.Generator().manual_seed(13)
    w = torch.randint(-64, 65, (M, Kd), generator=g).float() / 64.0   # 7 significant bits: one bf16 term holds it
    x = (torch.rand((S, Kd, Lp), generator=g) < 0.3).float()
    want = torch.einsum("mk,skl->sml", w.double(), x.double()).float()   # sums of multiples of 1/64 below 2^24 / 64: exact
    for wt, xt in ((3, 1), (2, 1), (1, 1), (3, 3)):
        got = C.pw_gemm(C.split_weight(w.cuda(), False), wt, M, Kd, x.cuda(), xt).cpu()
        assert torch.equal(got, want), (wt, xt)


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (1, 7, 3, 4), (4, 130, 257, 36), (16, 1152, 384, 196), (5, 384, 384, 196), (3, 70, 33, 6),
                                       (5, 200, 64, 198)])
@pytest.mark.parametrize("terms", [(3, 3), (3, 1), (1, 1)])
def test_gemm_leaves_the_batch_norm_sums_of_its_output(C, S, M, Kd, Lp, terms):
    """``pw_gemm(..., stats=True)``: the output is the one of the plain call bit for bit, and the partial sums add up to
    the per-channel sum and sum of squares of that output (float64 sums of the fp32 output; fp32 partial sums over 64
    columns each: 1e-6 of the sums of absolute values), so that the affine map made from them is the one ``bn_stats``
    gives."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    wt, xt = terms
    w = seeded_randn((M, Kd), 31, 0.0, 1.0)
    x = (seeded_randn((S, Kd, Lp), 32, 0.0, 1.0) > 0.3).float() if xt == 1 else seeded_randn((S, Kd, Lp), 32, 0.1, 1.0)
    planes = C.split_weight(w.cuda(), False)
    plain = C.pw_gemm(planes, wt, M, Kd, x.cuda(), xt)
    got, partial = C.pw_gemm(planes, wt, M, Kd, x.cuda(), xt, stats=True)
    assert torch.equal(got, plain)
    assert partial.shape == (L.load().sjhip_pwconv_gemm_stats_rows(Kd, S, Lp), M, 2)
    y = got.double()
    sums = partial.double().sum(0).cpu()
    want_s, want_q = y.sum((0, 2)).cpu(), (y * y).sum((0, 2)).cpu()
    abs_s = y.abs().sum((0, 2)).cpu().clamp_min(1e-30)
    assert float(((sums[:, 0] - want_s).abs() / abs_s).max()) < 1e-6
    assert float(((sums[:, 1] - want_q).abs() / want_q.clamp_min(1e-30)).max()) < 1e-6
    if Lp % 4 != 0:
        return  # (the pass over y of the batch-norm kernels takes rows of whole quads only)
    # the affine map from these sums against the one from the pass over y
    gamma, beta = seeded_randn((M,), 33, 1.0, 0.2).cuda(), seeded_randn((M,), 34, 0.0, 0.2).cuda()
    a = C._bn_map(got, gamma, beta, None, None, True, 0.1, 1e-5)
    b = C._bn_map(got, gamma, beta, None, None, True, 0.1, 1e-5, partial)
    torch.testing.assert_close(b[2], a[2], rtol=1e-6, atol=1e-6)      # mean
    torch.testing.assert_close(b[3], a[3], rtol=2e-6, atol=0.0)       # 1 / sqrt(var + eps)
    torch.testing.assert_close(b[0], a[0], rtol=2e-6, atol=0.0)
    torch.testing.assert_close(b[1], a[1], rtol=1e-5, atol=2e-6)


def test_gemm_over_several_launches(C):
    """Per-lane offsets into the activations are 32-bit byte offsets, so a call whose samples span more than 2^30 bytes
    of ``K * L`` rows runs as several launches over groups of samples (4095 samples of [4096, 64] fp32 and 5 more here): the
    output and the batch-norm sums must come out as for one launch.  Binary activations and weights that are multiples
    of 1/64 make every sum of the output exact, so that comparison is exact; samples are compared in slices to bound the
    memory."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    S, M, Kd, Lp = 4100, 8, 4096, 64
    g = torch.Generator(device="cuda").manual_seed(41)
    w = (torch.randint(-64, 65, (M, Kd), generator=torch.Generator().manual_seed(42)).float() / 64.0).cuda()
    x = (torch.rand((S, Kd, Lp), device="cuda", generator=g) < 0.05).float()
    planes = C.split_weight(w, False)
    got, partial = C.pw_gemm(planes, 3, M, Kd, x, 1, stats=True)
    rows = L.load().sjhip_pwconv_gemm_stats_rows(Kd, S, Lp)
    assert rows == 2 * (-(-4095 * Lp // 128)) + 2 * (-(-5 * Lp // 128)) and partial.shape == (rows, M, 2)
    for s0 in range(0, S, 410):
        want = torch.einsum("mk,skl->sml", w.double(), x[s0:s0 + 410].double()).float()
        assert torch.equal(got[s0:s0 + 410], want), s0
    sums = partial.double().sum(0)
    assert torch.equal(sums[:, 0], got.double().sum((0, 2)))
    want_q = (got.double() ** 2).sum((0, 2))   # the squares' fp32 partial sums are rounded: 1e-6
    assert float(((sums[:, 1] - want_q).abs() / want_q).max()) < 1e-6


# ---- the same GEMMs on two fp16 terms of scaled operands -----------------------------------------------------------
def _wide(shape, seed, decades, overall):
    """Normal values whose rows (second to last index) are spread over ``decades`` decades, times ``overall``."""
    base = seeded_randn(shape, seed, 0.05, 1.0)
    spread = 10.0 ** (seeded_randn(shape[:-1] + (1,), seed + 1000, 0.0, 1.0).clamp(-1.5, 1.5) * decades / 3.0)
    return base * spread * overall


@pytest.mark.parametrize("S,M,Kd,Lp", SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("w_scale,x_scale", [(1.0, 1.0), (3e-2, 1e-6), (1e-20, 1e12)])
def test_gemm_with_two_fp16_terms_has_fp32_accuracy(C, S, M, Kd, Lp, transpose, w_scale, x_scale):
    """Operands spread over four decades per tensor and placed anywhere in the fp32 range: the error stays within the
    bound of an fp32 dot product (the same bound as the three-term bf16 test), and is on average a few 2^-24 of
    ``sum |a||b|``."""
    F = C.F16 | 2
    w = _wide((Kd, M) if transpose else (M, Kd), 11, 4.0, w_scale)
    x = _wide((S, Kd, Lp), 12, 4.0, x_scale)
    planes = C.split_weight(w.cuda(), transpose, F)
    got = C.pw_gemm(planes, F, M, Kd, x.cuda(), F).cpu().double()
    a = (w.t() if transpose else w).double()
    want = torch.einsum("mk,skl->sml", a, x.double())
    bound = torch.einsum("mk,skl->sml", a.abs(), x.double().abs()).clamp_min(1e-300)
    rel = (got - want).abs() / bound
    assert torch.isfinite(got).all()
    assert float(rel.max()) < 2e-6
    assert float(rel.mean()) < 2e-7
    # the largest magnitude handed in is the one found inside; twice as much is still safe (one bit less headroom used)
    assert torch.equal(C.pw_gemm(planes, F, M, Kd, x.cuda(), F, False, C.amax(x.cuda())).cpu().double(), got)
    got2 = C.pw_gemm(planes, F, M, Kd, x.cuda(), F, False, C.amax(x.cuda()) * 2.0).cpu().double()
    assert float(((got2 - want).abs() / bound).max()) < 2e-6


def _column_errors(got, w, x):
    """Per output element: |got - float64| over the sum of |a||b| of its dot product."""
    want = torch.einsum("mk,skl->sml", w.double(), x.double())
    bound = torch.einsum("mk,skl->sml", w.double().abs(), x.double().abs()).clamp_min(1e-300)
    return (got.cpu().double() - want).abs() / bound


@pytest.mark.parametrize("S,M,Kd,Lp", [(24, 130, 96, 36), (16, 384, 384, 196)])
@pytest.mark.parametrize("what", ["samples", "outlier"])
def test_fp16_gemm_keeps_fp32_accuracy_over_a_wide_dynamic_range(C, S, M, Kd, Lp, what):
    """Activations (or gradients) whose samples are spread over eight decades (a batch in which some samples have
    converged), and a tensor with one element a million times the rest: every output column stays within 2e-6 of its
    own sum of |a||b|, because every sample is scaled by its own largest magnitude (with one scale per tensor a sample
    six decades below the largest would keep 2^-19 of relative accuracy, an eight-decade one 2^-12)."""
    F = C.F16 | 2
    w = seeded_randn((M, Kd), 93, 0.0, 0.05)
    x = seeded_randn((S, Kd, Lp), 94, 0.0, 1.0)
    if what == "samples":
        x = x * 10.0 ** torch.linspace(-8.0, 0.0, S)[:, None, None]
    else:
        x[S // 3, Kd // 2, Lp // 2] = 1e6
    planes = C.split_weight(w.cuda(), False, F)
    rel = _column_errors(C.pw_gemm(planes, F, M, Kd, x.cuda(), F), w, x)
    assert float(rel.max()) < 2e-6, float(rel.max())
    # the weight gradient sums over the samples: the tensor's scale, and what small samples add is small beside the rest
    # (holds when the samples that are small in one operand are not the only large ones in the other: gradients that
    # fade with the samples they belong to, against activations of any spread)
    dy = seeded_randn((S, M, Lp), 95, 0.0, 1.0)
    if what == "samples":
        dy = dy * 10.0 ** torch.linspace(-8.0, 0.0, S)[:, None, None]
    for xs in (x, seeded_randn((S, Kd, Lp), 98, 0.0, 1.0)):
        got = C.pw_grad_weight(dy.cuda(), F, xs.cuda(), F).cpu().double()
        want = torch.einsum("sml,snl->mn", dy.double(), xs.double())
        bound = torch.einsum("sml,snl->mn", dy.double().abs(), xs.double().abs())
        assert float(((got - want).abs() / bound).max()) < 2e-6
    # and the gradient with respect to the input, whose columns are samples again
    planes_t = C.split_weight(w.cuda(), True, F)
    rel = _column_errors(C.pw_gemm(planes_t, F, Kd, M, dy.cuda(), F), w.t(), dy)
    assert float(rel.max()) < 2e-6, float(rel.max())


@pytest.mark.parametrize("split", ["bf16", "f16"])
def test_gemm_with_token_columns_spread_over_eight_decades(C, split):
    """Positions of one sample spread over eight decades: the three-term bf16 split (fp32's exponent range) keeps every
    column within the fp32 bound; the fp16 split, whose scale is per sample, keeps the bound for columns above 2^-17 of
    their sample's largest magnitude and an absolute floor of 2^-38 of that magnitude times sum |a| below."""
    S, M, Kd, Lp = 4, 130, 96, 64
    F = C.F16 | 2 if split == "f16" else 3
    w = seeded_randn((M, Kd), 96, 0.0, 0.05)
    x = seeded_randn((S, Kd, Lp), 97, 0.0, 1.0) * 10.0 ** torch.linspace(-8.0, 0.0, Lp)[None, None, :]
    planes = C.split_weight(w.cuda(), False, F)
    got = C.pw_gemm(planes, F, M, Kd, x.cuda(), F).cpu().double()
    want = torch.einsum("mk,skl->sml", w.double(), x.double())
    bound = torch.einsum("mk,skl->sml", w.double().abs(), x.double().abs())
    err = (got - want).abs()
    if split == "bf16":
        assert float((err / bound).max()) < 2e-6
    else:
        floor = 2.0 ** -38 * x.double().abs().amax(dim=(1, 2))[:, None, None] * w.double().abs().sum(dim=1)[None, :, None]
        assert bool((err <= 2e-6 * bound + floor).all())
        large = (x.abs().amax(dim=1, keepdim=True) >= 2.0 ** -16 * x.abs().amax(dim=(1, 2), keepdim=True)).expand(S, M, Lp)
        assert float((err / bound)[large].max()) < 2e-6


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (4, 384, 384, 196)])
def test_fp16_gemm_is_exact_on_spikes_times_dyadic_weights(C, S, M, Kd, Lp):
    g = torch.Generator().manual_seed(13)
    w = torch.randint(-64, 65, (M, Kd), generator=g).float() / 64.0
    w = w * 2.0 ** torch.randint(-30, 20, (M, 1), generator=g).float()   # any power of two per row: the row scale takes it out
    x = (torch.rand((S, Kd, Lp), generator=g) < 0.3).float()
    want = torch.einsum("mk,skl->sml", w.double(), x.double()).float()
    F = C.F16 | 2
    planes = C.split_weight(w.cuda(), False, F)
    assert torch.equal(C.pw_gemm(planes, F, M, Kd, x.cuda(), C.F16 | 1).cpu(), want)
    assert torch.equal(C.pw_gemm(planes, F, M, Kd, x.cuda(), F).cpu(), want)
    zero = C.pw_gemm(planes, F, M, Kd, torch.zeros_like(x).cuda(), F)
    assert torch.equal(zero, torch.zeros_like(zero))
    planes0 = C.split_weight(torch.zeros_like(w).cuda(), False, F)
    assert not C.pw_gemm(planes0, F, M, Kd, x.cuda(), F).any()


def test_fp16_gemm_with_an_infinity_in_the_activations(C):
    """An infinity (or NaN) takes no part in the scale: the outputs that do not touch it are as accurate as without it,
    those that do are non-finite as in fp32."""
    F = C.F16 | 2
    S, M, Kd, Lp = 2, 40, 24, 8
    w = seeded_randn((M, Kd), 71, 0.0, 1.0)
    x = seeded_randn((S, Kd, Lp), 72, 0.0, 3e4)   # finite values beyond fp16's range when left unscaled
    x[1, 5, 3] = float("inf")
    x[0, 2, 6] = float("nan")
    got = C.pw_gemm(C.split_weight(w.cuda(), False, F), F, M, Kd, x.cuda(), F).cpu().double()
    want = torch.einsum("mk,skl->sml", w.double(), x.double())
    touched = torch.zeros((S, Lp), dtype=torch.bool)
    touched[1, 3] = touched[0, 6] = True
    clean = ~touched[:, None, :].expand(S, M, Lp)
    assert not torch.isfinite(got[~clean]).any()
    bound = torch.einsum("mk,skl->sml", w.double().abs(), torch.nan_to_num(x.double(), nan=0.0, posinf=0.0).abs())
    assert float(((got - want).abs() / bound)[clean].max()) < 2e-6


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (1, 7, 6, 4), (4, 130, 258, 36), (16, 384, 384, 196), (5, 1152, 384, 196)])
def test_fp16_gemms_read_bit_packed_spikes(C, S, M, Kd, Lp):
    """The GEMMs that take a spike tensor as bits give the results of the fp32-spike calls bit for bit: the forward with
    its batch-norm sums, and the weight gradient."""
    from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress

    F = C.F16 | 2
    w = _wide((M, Kd), 81, 2.0, 0.1).cuda()
    x = (seeded_randn((S, Kd, Lp), 82, 0.0, 1.0) > 0.4).float().cuda()
    bits = bit_spike_compress(x)
    planes = C.split_weight(w, False, F)
    want, want_partial = C.pw_gemm(planes, F, M, Kd, x, C.F16 | 1, stats=True)
    got, partial = C.pw_gemm_bits(planes, M, Kd, bits, S, Lp, stats=True)
    assert torch.equal(got, want) and torch.equal(partial, want_partial)
    assert torch.equal(C.pw_gemm_bits(planes, M, Kd, bits, S, Lp), want)
    dy = _wide((S, M, Lp), 83, 3.0, 1e-3).cuda()
    assert torch.equal(C.pw_grad_weight_bits(dy, bits, Kd), C.pw_grad_weight(dy, F, x, C.F16 | 1))


def test_amax(C):
    """``amax(x)``: the maximum of the first 256 words is the largest magnitude among the numbers of ``x``, for any length
    and alignment, ``sample_amax`` of the words that of every sample, and both fold into what the words already hold."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    for n, top in ((1, 1.0), (7, 3.0), (1000, 0.75), (4099, 1e-30), (1 << 20, 262016.0), (5, 0.0), (3 * (1 << 20) + 5, 17.5)):
        x = seeded_randn((n + 1,), n, 0.0, 1.0).clamp(-1, 1) * (top if top != 0.0 else 1.0) * 0.99
        if top == 0.0:
            x.zero_()
        x[n // 2 + 1] = -top
        top = abs(float(x[n // 2 + 1]))   # as fp32 holds it
        got = C.amax(x.cuda()[1:])        # one sample
        assert got.numel() == C.amax_floats(1) and float(got[:256].max()) == top == float(C.sample_amax(got)), (n, top)
        words = torch.zeros(C.amax_floats(1), device="cuda")   # the C entry point on an address 4 bytes past an aligned one
        xs = x.cuda()[1:]
        L.check(L.load().sjhip_pwconv_amax(xs.data_ptr(), 1, n, words.data_ptr(), L.current_stream_ptr(xs.device)), "amax")
        assert float(words.max()) == top and float(words.min()) >= 0.0
        words[3] = 1e30
        L.check(L.load().sjhip_pwconv_amax(xs.data_ptr(), 1, n, words.data_ptr(), L.current_stream_ptr(xs.device)), "amax")
        assert float(words[:256].max()) == max(top, float(torch.tensor(1e30))) and float(C.sample_amax(words)) == top
    odd = torch.tensor([1.0, float("nan"), -2.0, 0.5, float("-inf"), float("inf")]).cuda()
    assert float(C.amax(odd).max()) == 2.0   # the largest magnitude among the finite elements


@pytest.mark.parametrize("S,per_sample,offset", [(5, 12, 0), (3, 75264, 0), (300, 40, 0), (7, 4100, 0), (6, 10, 1), (4, 5000, 1),
                                                 (70000, 4, 0)])
def test_amax_per_sample(C, S, per_sample, offset):
    """Samples shorter and longer than the 4096 elements a block takes, sample lengths that are no multiple of 4 and a
    tensor that starts 4 bytes past an aligned address: every sample's word holds that sample's largest magnitude."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    x = seeded_randn((S * per_sample + offset,), 91, 0.0, 1.0)
    x = (x[offset:].view(S, per_sample) * (10.0 ** (seeded_randn((S, 1), 92, 0.0, 3.0)))).contiguous()
    x[S // 2] = 0.0
    flat = torch.empty(S * per_sample + offset, device="cuda")
    flat[offset:] = x.flatten().cuda()
    xd = flat[offset:].view(S, per_sample)
    words = torch.zeros(C.amax_floats(S), device="cuda")
    L.check(L.load().sjhip_pwconv_amax(xd.data_ptr(), S, per_sample, words.data_ptr(), L.current_stream_ptr(xd.device)), "amax")
    assert torch.equal(C.sample_amax(words).cpu(), x.abs().amax(dim=1))
    assert float(words[:256].max()) == float(x.abs().max())
    if offset == 0:
        assert torch.equal(C.sample_amax(C.amax(xd)), C.sample_amax(words))


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (1, 7, 3, 4), (4, 130, 257, 36), (16, 1152, 384, 196), (3, 70, 33, 6), (5, 200, 64, 198)])
@pytest.mark.parametrize("spikes", [False, True])
def test_fp16_gemm_leaves_the_batch_norm_sums_of_its_output(C, S, M, Kd, Lp, spikes):
    F = C.F16 | 2
    xt = C.F16 | 1 if spikes else F
    w = _wide((M, Kd), 31, 2.0, 0.1)
    x = (seeded_randn((S, Kd, Lp), 32, 0.0, 1.0) > 0.3).float() if spikes else _wide((S, Kd, Lp), 32, 2.0, 5.0)
    planes = C.split_weight(w.cuda(), False, F)
    plain = C.pw_gemm(planes, F, M, Kd, x.cuda(), xt)
    got, partial = C.pw_gemm(planes, F, M, Kd, x.cuda(), xt, stats=True)
    assert torch.equal(got, plain)
    y = got.double()
    sums = partial.double().sum(0).cpu()
    want_s, want_q = y.sum((0, 2)).cpu(), (y * y).sum((0, 2)).cpu()
    abs_s = y.abs().sum((0, 2)).cpu().clamp_min(1e-30)
    assert float(((sums[:, 0] - want_s).abs() / abs_s).max()) < 1e-6
    assert float(((sums[:, 1] - want_q).abs() / want_q.clamp_min(1e-30)).max()) < 1e-6


@pytest.mark.parametrize("S,M,N,Lp", [(3, 100, 50, 12), (9, 130, 257, 36), (16, 384, 384, 196), (2, 1152, 384, 196), (64, 64, 48, 8)])
@pytest.mark.parametrize("spikes", [False, True])
@pytest.mark.parametrize("dy_scale", [1.0, 1e-9])
def test_fp16_grad_weight_gemm(C, S, M, N, Lp, spikes, dy_scale):
    F = C.F16 | 2
    dy = _wide((S, M, Lp), 21, 4.0, dy_scale)
    x = (seeded_randn((S, N, Lp), 22, 0.0, 1.0) > 0.5).float() if spikes else _wide((S, N, Lp), 22, 4.0, 30.0)
    got = C.pw_grad_weight(dy.cuda(), F, x.cuda(), C.F16 | 1 if spikes else F).cpu().double()
    want = torch.einsum("sml,snl->mn", dy.double(), x.double())
    bound = torch.einsum("sml,snl->mn", dy.double().abs(), x.double().abs()).clamp_min(1e-300)
    rel = (got - want).abs() / bound
    assert float(rel.max()) < 2e-6 and float(rel.mean()) < 2e-7


# ---- operands that arrive as fp16 term planes (split once by their producer, not by every block of a GEMM) ---------------
PLANE_SHAPES = [(3, 100, 50, 12), (2, 128, 32, 128), (1, 7, 3, 4), (4, 130, 257, 36), (5, 384, 384, 196), (16, 1152, 384, 196),
                (3, 40, 9, 20)]


@pytest.mark.parametrize("S,M,Kd,Lp", PLANE_SHAPES)
@pytest.mark.parametrize("x_scale", [1.0, 1e-6, 1e12])
def test_plane_layout_is_the_split_of_the_scaled_tensor(C, S, M, Kd, Lp, x_scale):
    """``split_planes``: plane 0 is fp16(scale x), plane 1 fp16 of the remainder, rows of channels with the columns of all
    samples in a row; scale = the power of two that takes amax into [2^14, 2^15)."""
    x = _wide((S, Kd, Lp), 31, 4.0, x_scale).cuda()
    xa = C.amax(x)
    planes = C.split_planes(x, xa)
    ld = -(-S * Lp // 8) * 8
    assert planes.numel() == 2 * Kd * ld
    top = float(xa.max())
    scale = 2.0 ** (14 - int(torch.tensor(top).log2().floor()))
    xs = (x.double() * scale).permute(1, 0, 2).reshape(Kd, S * Lp)
    hi = planes[:Kd * ld].view(Kd, ld)[:, :S * Lp]
    lo = planes[Kd * ld:].view(Kd, ld)[:, :S * Lp]
    assert torch.equal(hi, xs.float().half())
    assert torch.equal(lo, (xs.float() - hi.float()).half())
    # two terms hold 22 significant bits of a value, down to the subnormal spacing 2^-24 of the second
    assert bool(((hi.double() + lo.double() - xs).abs() <= xs.abs() * 2.0 ** -22 + 2.0 ** -25).all())


@pytest.mark.parametrize("S,M,Kd,Lp", PLANE_SHAPES)
@pytest.mark.parametrize("transpose", [False, True])
def test_gemm_from_planes_has_fp32_accuracy_and_leaves_the_batch_norm_sums(C, S, M, Kd, Lp, transpose):
    F = C.F16 | 2
    w = _wide((Kd, M) if transpose else (M, Kd), 32, 4.0, 0.05)
    x = _wide((S, Kd, Lp), 33, 4.0, 3.0)
    wp = C.split_weight(w.cuda(), transpose, F)
    xa = C.amax(x.cuda())
    xp = C.split_planes(x.cuda(), xa)
    got, part = C.pw_gemm_planes(wp, M, Kd, xp, 2, xa, S, Lp, True)
    assert torch.equal(C.pw_gemm_planes(wp, M, Kd, xp, 2, xa, S, Lp), got)
    got = got.cpu().double()
    a = (w.t() if transpose else w).double()
    want = torch.einsum("mk,skl->sml", a, x.double())
    bound = torch.einsum("mk,skl->sml", a.abs(), x.double().abs()).clamp_min(1e-300)
    rel = (got - want).abs() / bound
    assert torch.isfinite(got).all() and float(rel.max()) < 2e-6 and float(rel.mean()) < 2e-7
    # the same operands through the kernels that split while they stage: equal up to the fp32 accumulation order
    ref = C.pw_gemm(wp, F, M, Kd, x.cuda(), F, False, xa).cpu().double()
    assert float(((got - ref).abs() / bound).max()) < 1e-6
    sums = part.double().sum(0).cpu()
    want_s, abs_s, want_q = got.sum((0, 2)), got.abs().sum((0, 2)).clamp_min(1e-30), (got ** 2).sum((0, 2))
    assert float(((sums[:, 0] - want_s).abs() / abs_s).max()) < 1e-6
    assert float(((sums[:, 1] - want_q).abs() / want_q.clamp_min(1e-30)).max()) < 1e-6


@pytest.mark.parametrize("S,M,Kd,Lp", [(3, 100, 50, 12), (4, 384, 384, 196)])
def test_gemm_from_a_plane_of_spikes_is_exact(C, S, M, Kd, Lp):
    g = torch.Generator().manual_seed(34)
    w = torch.randint(-64, 65, (M, Kd), generator=g).float() / 64.0
    x = (torch.rand((S, Kd, Lp), generator=g) < 0.3).float()
    wp = C.split_weight(w.cuda(), False, C.F16 | 2)
    xp = C.split_planes(x.cuda(), None, 1)
    got = C.pw_gemm_planes(wp, M, Kd, xp, 1, None, S, Lp)
    assert torch.equal(got.cpu().double(), torch.einsum("mk,skl->sml", w.double(), x.double()))


@pytest.mark.parametrize("S,M,N,Lp", [(3, 100, 50, 12), (9, 130, 257, 36), (16, 384, 384, 196), (2, 1152, 384, 196), (64, 64, 48, 8),
                                      (1, 5, 3, 4)])
@pytest.mark.parametrize("spikes", [False, True])
def test_grad_weight_from_planes(C, S, M, N, Lp, spikes):
    dy = _wide((S, M, Lp), 35, 4.0, 1e-3)
    x = (seeded_randn((S, N, Lp), 36, 0.0, 1.0) > 0.5).float() if spikes else _wide((S, N, Lp), 36, 4.0, 30.0)
    dya = C.amax(dy.cuda())
    xa = None if spikes else C.amax(x.cuda())
    dyp, xp = C.split_planes(dy.cuda(), dya), C.split_planes(x.cuda(), xa, 1 if spikes else 2)
    got = C.pw_grad_weight_planes(dyp, dya, xp, 1 if spikes else 2, xa, S, M, N, Lp).cpu().double()
    want = torch.einsum("sml,snl->mn", dy.double(), x.double())
    bound = torch.einsum("sml,snl->mn", dy.double().abs(), x.double().abs()).clamp_min(1e-300)
    rel = (got - want).abs() / bound
    assert float(rel.max()) < 2e-6 and float(rel.mean()) < 2e-7


def test_plane_calls_refuse_what_they_cannot_run(C):
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    x = torch.randn(2, 8, 6, device="cuda")  # rows of six positions: not a multiple of 4
    with pytest.raises(RuntimeError, match="multiple of 4"):
        C.split_planes(x, C.amax(x))
    x = torch.randn(2, 8, 8, device="cuda")
    with pytest.raises(RuntimeError, match="amax"):
        C.split_planes(x, None, 2)
    assert L.load().sjhip_pwconv_plane_elems(2, 8, 8, 3) == 0


@pytest.mark.parametrize("S,Cc,Lp", [(3, 5, 12), (16, 384, 196), (7, 33, 4), (300, 64, 100)])
def test_bn_grad_input_leaves_the_largest_magnitude_of_its_output(C, S, Cc, Lp):
    """``sjhip_bn_grad_input_amax``: the same ``dy`` as the plain call, and the largest magnitude a pass over it finds."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    lib = L.load()
    g = (seeded_randn((S, Cc, Lp), 51, 0.0, 1.0) * 1e-4).cuda()
    y = seeded_randn((S, Cc, Lp), 52, 0.3, 2.0).cuda()
    coef = seeded_randn((3, Cc), 53, 0.0, 1.0).cuda()
    plain, fused = torch.empty_like(g), torch.empty_like(g)
    word = torch.zeros((C.amax_floats(S),), dtype=torch.float32, device="cuda")
    stream = L.current_stream_ptr(g.device)
    L.check(lib.sjhip_bn_grad_input(g.data_ptr(), y.data_ptr(), coef.data_ptr(), S, Cc, Lp, plain.data_ptr(), stream), "plain")
    L.check(lib.sjhip_bn_grad_input_amax(g.data_ptr(), y.data_ptr(), coef.data_ptr(), S, Cc, Lp, fused.data_ptr(),
                                         word.data_ptr(), stream), "fused")
    assert torch.equal(plain, fused)
    assert float(word[:256].max()) == float(plain.abs().max())
    assert torch.equal(C.sample_amax(word), plain.abs().amax(dim=(1, 2)))   # every sample's own largest magnitude
    assert torch.equal(C.sample_amax(C.amax(plain)), C.sample_amax(word))


def test_launches_that_clear_an_amax_buffer_and_count_the_batch(C):
    """The fp16 weight split and the batch-norm backward's coefficient kernel set a given amax buffer to zero (so that the
    launch that folds the maxima next needs no fill in front of it); the batch-norm forward's finalize adds 1 to the
    counter of batches."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    for samples in (0, 5, 1000):
        buf = torch.full((C.amax_floats(samples),), 1e30, device="cuda")
        C.split_weight(seeded_randn((40, 24), 61, 0.0, 1.0).cuda(), False, C.F16 | 2, buf)
        assert not buf.any()
    T, B, Cc, Lp = 4, 3, 10, 12
    y = seeded_randn((T, B, Cc, Lp), 62, 0.4, 1.5).cuda()
    gamma, beta = seeded_randn((Cc,), 63, 1.0, 0.2).cuda(), seeded_randn((Cc,), 64, 0.6, 0.3).cuda()
    tracked = torch.tensor(41, dtype=torch.int64, device="cuda")
    bn_map = C._bn_map(y.flatten(0, 1), gamma, beta, None, None, True, 0.1, 1e-5, None, tracked)
    assert int(tracked) == 42
    spec = (2.0, 1.0, 0.0, K._flags(False, False, True, 0), no.SG_IDS["sigmoid"], no.SG_DEFAULT_ALPHA["sigmoid"])
    v0 = torch.zeros((1,), device="cuda").expand(B, Cc, Lp)
    gs = seeded_randn((T, B, Cc, Lp), 65).cuda()
    for _ in range(3):   # the buffer comes from torch.empty: whatever it held before must not survive
        poison = torch.full((C.amax_floats(T * B),), 1e30, device="cuda")
        del poison
        dy, _, _, _, dy_amax = C._bn_lif_backward(y, bn_map, gamma, v0, spec, True, gs, None, False, True)
        assert float(dy_amax[:256].max()) == float(dy.abs().max())
        assert torch.equal(C.sample_amax(dy_amax), dy.abs().amax(dim=(2, 3)).flatten())
    plain = C._bn_lif_backward(y, bn_map, gamma, v0, spec, True, gs, None, False)[0]
    assert torch.equal(plain, dy)


@pytest.mark.parametrize("S,M,N,Lp", [(3, 100, 50, 12), (9, 130, 257, 36), (16, 384, 384, 196), (2, 1152, 384, 196), (64, 64, 48, 8)])
@pytest.mark.parametrize("spikes", [False, True])
def test_grad_weight_gemm(C, S, M, N, Lp, spikes):
    dy = seeded_randn((S, M, Lp), 21, 0.0, 1.0)
    x = (seeded_randn((S, N, Lp), 22, 0.0, 1.0) > 0.5).float() if spikes else seeded_randn((S, N, Lp), 22, 0.2, 1.0)
    got = C.pw_grad_weight(dy.cuda(), 3, x.cuda(), 1 if spikes else 3).cpu().double()
    want = torch.einsum("sml,snl->mn", dy.double(), x.double())
    bound = torch.einsum("sml,snl->mn", dy.double().abs(), x.double().abs()).clamp_min(1e-30)
    assert float(((got - want).abs() / bound).max()) < 2e-6


# ------------------------------------------------------------------------------------------------
# batch norm + LIF
# ------------------------------------------------------------------------------------------------
def _no_borderline(h, v_th):
    """No membrane potential within the margin of the threshold.  Exact ties are allowed: they occur in the attention
    neuron, whose inputs are multiples of 1/8 and whose arithmetic is therefore exact in fp32 and float64 alike."""
    d = (h - v_th).abs()
    return bool(((d > MARGIN) | (d == 0)).all())


# (more than 16 steps: the backward walks the sequence in pieces of 16, one kernel variant per row shape)
@pytest.mark.parametrize("T,B,Cc,Lp", [(4, 3, 10, 12), (1, 2, 5, 4), (7, 2, 33, 20), (16, 2, 6, 260), (4, 2, 12, 196),
                                       (17, 2, 5, 36), (33, 1, 6, 196), (40, 1, 3, 260), (64, 2, 3, 8), (256, 1, 2, 196), (250, 1, 3, 16)])
@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("v_reset,decay_input,tau,sg", [(0.0, True, 2.0, "sigmoid"), (None, False, 3.0, "atan"), (-0.2, True, 2.5, "erf")])
def test_bn_lif_against_float64(C, T, B, Cc, Lp, training, v_reset, decay_input, tau, sg):
    from spikingjelly_amd.activation_based.hip_kernel import library as L
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    gamma, beta = seeded_randn((Cc,), 32, 1.0, 0.2), seeded_randn((Cc,), 33, 0.6, 0.3)
    rm, rv = seeded_randn((Cc,), 34, 0.3, 0.2), seeded_randn((Cc,), 35, 2.0, 0.3).abs()
    gs = seeded_randn((T, B, Cc, Lp), 36)
    gl = seeded_randn((B, Cc, Lp), 37, 0.0, 0.3)
    alpha = no.SG_DEFAULT_ALPHA[sg]
    detach = v_reset is None
    for seed in range(31, 3100, 100):  # the first input whose membrane potentials all keep the margin from the threshold
        y = seeded_randn((T, B, Cc, Lp), seed, 0.4, 1.5)
        y64 = y.double().requires_grad_()
        g64, b64 = gamma.double().requires_grad_(), beta.double().requires_grad_()
        z, rm64, rv64 = co.batch_norm(y64, g64, b64, rm.double(), rv.double(), training)
        s64, v64, h64 = co.lif(z, torch.full((B, Cc, Lp), 0.0 if v_reset is None else v_reset, dtype=torch.float64), tau, 1.0,
                               v_reset, detach, sg, alpha, decay_input)
        if _no_borderline(h64.detach(), 1.0):
            break
    else:
        pytest.fail("no input without a neuron within the margin of the threshold")
    torch.autograd.backward([s64, v64[-1]], [gs.double(), gl.double()])

    soft = v_reset is None
    flags = K._flags(soft, detach, decay_input, 0)
    spec = (tau, 1.0, 0.0 if soft else v_reset, flags, no.SG_IDS[sg], alpha)
    yd = y.cuda().requires_grad_()
    gd, bd = gamma.cuda().requires_grad_(), beta.cuda().requires_grad_()
    rmd, rvd = rm.cuda(), rv.cuda()
    v0 = torch.full((1,), 0.0 if soft else v_reset, device="cuda").expand(B, Cc, Lp)
    spikes, v_last = C.bn_lif(yd, gd, bd, v0, (rmd, rvd, training, 0.1, 1e-5), spec)
    torch.autograd.backward([spikes, v_last], [gs.cuda(), gl.cuda()])
    assert torch.equal(spikes.detach().cpu().double(), s64.detach())
    torch.testing.assert_close(v_last.detach().cpu().double(), v64[-1].detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(rmd.cpu().double(), rm64, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(rvd.cpu().double(), rv64, rtol=1e-6, atol=1e-6)
    scale = float(y64.grad.abs().max())
    torch.testing.assert_close(yd.grad.cpu().double(), y64.grad, rtol=1e-4, atol=1e-5 * scale)
    torch.testing.assert_close(gd.grad.cpu().double(), g64.grad, rtol=1e-4, atol=1e-5 * float(g64.grad.abs().max()))
    torch.testing.assert_close(bd.grad.cpu().double(), b64.grad, rtol=1e-4, atol=1e-5 * float(b64.grad.abs().max()))


@pytest.mark.parametrize("T,B,Cc,Lp", [(4, 3, 10, 12), (7, 2, 33, 20), (16, 2, 6, 260), (4, 2, 12, 196), (33, 1, 6, 196), (20, 2, 5, 36)])
@pytest.mark.parametrize("v_reset,decay_input,init_tau,sg", [(0.0, True, 2.0, "sigmoid"), (None, False, 3.0, "atan"), (-0.2, True, 2.5, "erf")])
def test_bn_plif_against_float64(C, T, B, Cc, Lp, v_reset, decay_input, init_tau, sg):
    """Batch norm + parametric LIF (``k = 1 / init_tau`` read from device memory): spikes, state and the gradients of
    the input, of the batch-norm parameters and of ``k`` against autograd through the float64 oracle
    (``neuron_oracle.multi_step('plif_k')``, restating functional/neuron.py:1215-1297)."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    gamma, beta = seeded_randn((Cc,), 132, 1.0, 0.2), seeded_randn((Cc,), 133, 0.6, 0.3)
    gs = seeded_randn((T, B, Cc, Lp), 136)
    gl = seeded_randn((B, Cc, Lp), 137, 0.0, 0.3)
    alpha = no.SG_DEFAULT_ALPHA[sg]
    detach = v_reset is None
    k32 = torch.tensor([1.0 / init_tau], dtype=torch.float32)
    start = 0.0 if v_reset is None else v_reset
    for seed in range(131, 3200, 100):  # the first input whose membrane potentials all keep the margin from the threshold
        y = seeded_randn((T, B, Cc, Lp), seed, 0.4, 1.5)
        y64 = y.double().requires_grad_()
        g64, b64 = gamma.double().requires_grad_(), beta.double().requires_grad_()
        k64 = k32.double().requires_grad_()
        z, _, _ = co.batch_norm(y64, g64, b64, torch.zeros(Cc, dtype=torch.float64), torch.ones(Cc, dtype=torch.float64), True)
        s64, v64, h64 = no.multi_step("plif_k", z.flatten(1), torch.full((B * Cc * Lp,), start, dtype=torch.float64), k64[0],
                                      decay_input, 1.0, v_reset, no.surrogate(sg, alpha), detach)
        if _no_borderline(h64.detach(), 1.0):
            break
    else:
        pytest.fail("no input without a neuron within the margin of the threshold")
    torch.autograd.backward([s64, v64[-1]], [gs.double().flatten(1), gl.double().flatten()])

    soft = v_reset is None
    spec = (0.0, 1.0, 0.0 if soft else v_reset, K._flags(soft, detach, decay_input, 0), no.SG_IDS[sg], alpha)
    yd = y.cuda().requires_grad_()
    gd, bd = gamma.cuda().requires_grad_(), beta.cuda().requires_grad_()
    kd = k32.cuda().requires_grad_()
    v0 = torch.full((1,), start, device="cuda").expand(B, Cc, Lp)
    spikes, v_last = C.bn_lif(yd, gd, bd, v0, (torch.zeros(Cc, device="cuda"), torch.ones(Cc, device="cuda"), True, 0.1, 1e-5),
                              spec, kd)
    torch.autograd.backward([spikes, v_last], [gs.cuda(), gl.cuda()])
    assert torch.equal(spikes.detach().cpu().double().flatten(1), s64.detach())
    torch.testing.assert_close(v_last.detach().cpu().double().flatten(), v64[-1].detach(), rtol=1e-5, atol=1e-5)
    scale = float(y64.grad.abs().max())
    torch.testing.assert_close(yd.grad.cpu().double(), y64.grad, rtol=1e-4, atol=1e-5 * scale)
    torch.testing.assert_close(gd.grad.cpu().double(), g64.grad, rtol=1e-4, atol=1e-5 * float(g64.grad.abs().max()))
    torch.testing.assert_close(bd.grad.cpu().double(), b64.grad, rtol=1e-4, atol=1e-5 * float(b64.grad.abs().max()))
    # dL/dk: a sum over every neuron-step (fp32 terms, fp64 reduction): 1e-4 of the sum of the terms' magnitudes is far
    # below what a dropped step, a wrong v[t-1] or a missing division by k would change
    assert float(kd.grad.cpu().double() - k64.grad) == pytest.approx(0.0, abs=1e-4 * max(1.0, float(k64.grad.abs())) + 1e-3)
    assert abs(float(k64.grad)) > 1e-2


@pytest.mark.parametrize("T,B,Cc,Lp", [(4, 3, 10, 12), (16, 2, 6, 260), (4, 2, 12, 196), (20, 2, 5, 36)])
@pytest.mark.parametrize("v_reset,sg", [(0.0, "sigmoid"), (None, "atan")])
def test_bn_if_against_float64(C, T, B, Cc, Lp, v_reset, sg):
    """Batch norm + IF neuron (a spec without a time constant) against the float64 oracle (functional/neuron.py:242-312)."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    gamma, beta = seeded_randn((Cc,), 232, 0.5, 0.1), seeded_randn((Cc,), 233, 0.3, 0.2)
    gs = seeded_randn((T, B, Cc, Lp), 236)
    alpha = no.SG_DEFAULT_ALPHA[sg]
    detach = v_reset is None
    start = 0.0 if v_reset is None else v_reset
    for seed in range(231, 3300, 100):
        y = seeded_randn((T, B, Cc, Lp), seed, 0.4, 1.5)
        y64, g64, b64 = y.double().requires_grad_(), gamma.double().requires_grad_(), beta.double().requires_grad_()
        z, _, _ = co.batch_norm(y64, g64, b64, torch.zeros(Cc, dtype=torch.float64), torch.ones(Cc, dtype=torch.float64), True)
        s64, v64, h64 = no.multi_step("if", z.flatten(1), torch.full((B * Cc * Lp,), start, dtype=torch.float64), None, False, 1.0,
                                      v_reset, no.surrogate(sg, alpha), detach)
        if _no_borderline(h64.detach(), 1.0):
            break
    else:
        pytest.fail("no input without a neuron within the margin of the threshold")
    s64.backward(gs.double().flatten(1))
    soft = v_reset is None
    spec = (0.0, 1.0, 0.0 if soft else v_reset, K._flags(soft, detach, False, 0), no.SG_IDS[sg], alpha)
    yd, gd, bd = y.cuda().requires_grad_(), gamma.cuda().requires_grad_(), beta.cuda().requires_grad_()
    v0 = torch.full((1,), start, device="cuda").expand(B, Cc, Lp)
    spikes, v_last = C.bn_lif(yd, gd, bd, v0, (torch.zeros(Cc, device="cuda"), torch.ones(Cc, device="cuda"), True, 0.1, 1e-5), spec)
    spikes.backward(gs.cuda())
    assert torch.equal(spikes.detach().cpu().double().flatten(1), s64.detach())
    torch.testing.assert_close(v_last.detach().cpu().double().flatten(), v64[-1].detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(yd.grad.cpu().double(), y64.grad, rtol=1e-4, atol=1e-5 * float(y64.grad.abs().max()))
    torch.testing.assert_close(gd.grad.cpu().double(), g64.grad, rtol=1e-4, atol=1e-5 * float(g64.grad.abs().max()))
    torch.testing.assert_close(bd.grad.cpu().double(), b64.grad, rtol=1e-4, atol=1e-5 * float(b64.grad.abs().max()))


def test_if_neuron_at_the_end_of_a_chain_runs_fused(monkeypatch):
    """``Conv1d(k=1) -> BatchNorm1d -> IFNode``: fused, and equal to the modules called one by one outside the margin."""
    from spikingjelly_amd.activation_based.layer import fused

    torch.manual_seed(5)
    conv, bn = nn.Conv1d(32, 48, 1, bias=False).cuda(), nn.BatchNorm1d(48).cuda()
    with torch.no_grad():
        bn.weight.fill_(0.6)
        bn.bias.fill_(0.3)
    node = neuron.IFNode(step_mode="m", backend="hip").cuda()
    x = seeded_randn((4, 3, 32, 36), 6, 0.0, 1.0).cuda()
    out = fused.conv_bn_lif(x.clone().requires_grad_(), conv, bn, node)
    assert out is not None and 0.02 < float(out.detach().mean()) < 0.9
    functional.reset_net(node)
    ref = node(bn(conv(x.flatten(0, 1))).view(4, 3, 48, 36))
    assert float((out.detach() != ref.detach()).float().mean()) < 1e-3


def test_parametric_lif_at_the_end_of_the_chains_runs_fused_and_trains_its_parameter(monkeypatch):
    """A block whose ``qkv_lif`` and ``proj_lif`` are ``ParametricLIFNode``s: both chains stay fused, the spikes are
    those of the unfused modules (torch's convolution and batch norm around the hip neurons) outside the margin, and
    ``w.grad`` of both neurons agrees with the unfused path."""
    from spikingjelly_amd.activation_based.layer import fused

    def make():
        block = _make_block(64, 2, 71)
        block.qkv_lif = neuron.ParametricLIFNode(init_tau=2.5, step_mode="m", backend="hip")
        block.proj_lif = neuron.ParametricLIFNode(init_tau=3.0, step_mode="m", backend="hip")
        return block.cuda().train()

    fused_block, plain_block = make(), make()
    ran, real_a, real_b = [], fused.conv_bn_lif, fused.lif_conv_bn_lif
    monkeypatch.setattr(fused, "conv_bn_lif", lambda *a, **k: (lambda r: ran.append(("qkv", r is not None)) or r)(real_a(*a, **k)))
    monkeypatch.setattr(fused, "lif_conv_bn_lif", lambda *a, **k: (lambda r: ran.append(("proj", r is not None)) or r)(real_b(*a, **k)))
    x = seeded_randn((4, 3, 64, 36), 72, 0.0, 2.0).cuda()
    g = seeded_randn((4, 3, 64, 36), 73).cuda()
    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", True)
    xa = x.clone().requires_grad_()
    out_a = fused_block(xa)
    out_a.backward(g)
    assert ("qkv", True) in ran and ("proj", True) in ran
    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", False)
    xb = x.clone().requires_grad_()
    out_b = plain_block(xb)
    out_b.backward(g)
    assert float((out_a.detach() != out_b.detach()).float().mean()) < 2e-3 and 0.02 < float(out_a.detach().mean()) < 0.9
    for name in ("qkv_lif", "proj_lif"):
        wa, wb = getattr(fused_block, name).w.grad, getattr(plain_block, name).w.grad
        assert wa is not None and abs(float(wb)) > 1e-4
        assert float(wa) == pytest.approx(float(wb), rel=5e-2, abs=1e-3)
    torch.testing.assert_close(xa.grad, xb.grad, rtol=5e-2, atol=5e-3 * float(xb.grad.abs().max()))


def test_bn_lif_bit_packed_spikes_equal_the_dense_ones(C):
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K
    from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress

    T, B, Cc, Lp = 4, 3, 10, 196   # rows of 196 spikes start in the middle of a byte every other row
    y = seeded_randn((T, B * 2, Cc, Lp), 41, 0.4, 1.5).cuda()
    beta = torch.full((Cc,), 0.8, device="cuda")
    bn_map = C._bn_map(y.flatten(0, 1), None, beta, None, None, True, 0.1, 1e-5)
    spec = (2.0, 1.0, 0.0, K._flags(False, True, True, 0), 0, 4.0)
    v0 = torch.zeros((B * 2, Cc, Lp), device="cuda")
    dense, v_a = C._bn_lif_forward(y, bn_map, v0, spec, False)
    bits, v_b = C._bn_lif_forward(y, bn_map, v0, spec, True)
    assert torch.equal(bits, bit_spike_compress(dense)) and torch.equal(v_a, v_b)
    assert 0.05 < float(dense.mean()) < 0.95


# ------------------------------------------------------------------------------------------------
# the whole chain and the attention block
# ------------------------------------------------------------------------------------------------
def _block_params(block):
    params = {}
    for name, seq in (("qkv", block.qkv_conv_bn), ("proj", block.proj_conv_bn)):
        params[f"{name}_weight"] = seq[0].weight.detach()[:, :, 0].double().cpu().clone().requires_grad_()
        params[f"{name}_gamma"] = seq[1].weight.detach().double().cpu().clone().requires_grad_()
        params[f"{name}_beta"] = seq[1].bias.detach().double().cpu().clone().requires_grad_()
        params[f"{name}_running_mean"] = seq[1].running_mean.double().cpu().clone()
        params[f"{name}_running_var"] = seq[1].running_var.double().cpu().clone()
    return params


def _make_block(dim, heads, seed):
    torch.manual_seed(seed)
    block = layer.SpikingSelfAttention(dim, heads, backend="hip")
    with torch.no_grad():
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.running_mean.normal_(0.0, 0.1)
            bn.running_var.uniform_(0.5, 1.5)
            bn.weight.normal_(1.0, 0.2)
            bn.bias.normal_(0.9, 0.3)
    return block


@pytest.mark.parametrize("dim,heads,T,B,tokens", [(16, 2, 3, 2, 8), (64, 2, 4, 2, 36), (48, 3, 4, 1, 196), (32, 2, 20, 1, 36)])
@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("split,overlap", [("f16", True), ("f16", False), ("bf16", True)])
def test_attention_block_fused_against_float64(dim, heads, T, B, tokens, training, split, overlap, monkeypatch):
    """Both splits of the convolution GEMMs' operands, and the two gradients of a convolution on two streams or one."""

    monkeypatch.setattr(configure, "hip_conv_split", split)
    monkeypatch.setattr(configure, "hip_conv_overlap_gradients", overlap)
    block = _make_block(dim, heads, 50 + dim).cuda().train(training)
    params = _block_params(block)
    g = seeded_randn((T, B, dim, tokens), 52)
    for seed in range(51, 5100, 100):  # the first input that keeps every neuron of the three layers off its threshold
        x = seeded_randn((T, B, dim, tokens), seed, 0.0, 2.0)
        x64 = x.double().requires_grad_()
        ref = co.attention_block(x64, params, heads, training)
        if all(_no_borderline(h.detach(), v_th) for h, v_th in ((ref["qkv_h"], 1.0), (ref["attn_h"], 0.5), (ref["proj_h"], 1.0))):
            break
    else:
        pytest.fail("no input without a neuron within the margin of a threshold")
    ref["out"].backward(g.double())

    xd = x.cuda().requires_grad_()
    out = block(xd)
    out.backward(g.cuda())
    assert torch.equal(out.detach().cpu().double(), ref["out"].detach())
    assert 0.02 < float(out.detach().mean()) < 0.9
    assert block.qkv_lif.v.shape == (B, 3 * dim, tokens) and block.proj_lif.v.shape == (B, dim, tokens)

    def close(a, b, what):
        scale = float(b.abs().max())
        torch.testing.assert_close(a.cpu().double(), b, rtol=1e-4, atol=2e-5 * scale, msg=lambda m: f"{what}: {m}")

    close(xd.grad, x64.grad, "grad x")
    for name, seq in (("qkv", block.qkv_conv_bn), ("proj", block.proj_conv_bn)):
        close(seq[0].weight.grad[:, :, 0], params[f"{name}_weight"].grad, name + " weight")
        close(seq[1].weight.grad, params[f"{name}_gamma"].grad, name + " gamma")
        close(seq[1].bias.grad, params[f"{name}_beta"].grad, name + " beta")
        if training:
            torch.testing.assert_close(seq[1].running_mean.cpu().double(), ref[f"{name}_running"][0], rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(seq[1].running_var.cpu().double(), ref[f"{name}_running"][1], rtol=1e-5, atol=1e-6)
            assert int(seq[1].num_batches_tracked) == 1


def test_convolution_gradients_on_two_streams_equal_those_on_one(monkeypatch):
    """The weight gradient on a second stream beside the input gradient: the same kernels on the same data, so the same
    bits, also when other work is queued behind them and the step is repeated."""

    block = _make_block(64, 2, 61).cuda().train()
    x = seeded_randn((4, 3, 64, 36), 62, 0.0, 2.0).cuda()
    g = seeded_randn((4, 3, 64, 36), 63).cuda()
    results = []
    for overlap in (False, True, True):
        monkeypatch.setattr(configure, "hip_conv_overlap_gradients", overlap)
        xi = x.clone().requires_grad_()
        for p_ in block.parameters():
            p_.grad = None
        functional.reset_net(block)
        out = block(xi)
        out.backward(g)
        busy = (xi.grad * 2.0).sum()   # work queued right behind the backward
        results.append([xi.grad.clone()] + [p_.grad.clone() for p_ in block.parameters()] + [busy])
    torch.cuda.synchronize()
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b)


@pytest.mark.parametrize("training", [True, False])
def test_bit_packed_spikes_between_attention_neuron_and_projection_change_nothing(training, monkeypatch):
    """``configure.hip_conv_bit_spikes``: the attention neuron writes bits and the projection's GEMMs read bits, or the
    spikes travel as fp32; the same arithmetic on the same values, so outputs, states and gradients are the same bits,
    over two consecutive calls (the second starts from the states of the first)."""
    block = _make_block(64, 2, 65).cuda().train(training)
    xs = [seeded_randn((4, 3, 64, 36), 66 + i, 0.0, 2.0).cuda() for i in range(2)]
    g = seeded_randn((4, 3, 64, 36), 68).cuda()
    results = []
    for bits in (False, True):
        monkeypatch.setattr(configure, "hip_conv_bit_spikes", bits)
        functional.reset_net(block)
        got = []
        for x in xs:
            for p_ in block.parameters():
                p_.grad = None
            xi = x.clone().requires_grad_()
            out = block(xi)
            out.backward(g)
            got += [out.detach().clone(), xi.grad.clone(), block.attn_lif.v.detach().clone(), block.proj_lif.v.detach().clone()]
            got += [p_.grad.clone() for p_ in block.parameters()]
            for node in (block.qkv_lif, block.attn_lif, block.proj_lif):   # the next call starts from these states
                node.v = node.v.detach()
        results.append(got)
    assert results[0][2].shape == results[1][2].shape == (3, 2, 32, 36)   # the attention neuron's state keeps its shape
    assert 0.02 < float(results[0][0].mean()) < 0.9
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_attention_block_fused_equals_unfused_path(monkeypatch):
    """The same module with the fusion switched off (torch's convolution and batch norm around the hip neurons)."""
    from spikingjelly_amd.activation_based.layer import fused

    block = _make_block(64, 2, 60).cuda().train()
    x = seeded_randn((4, 2, 64, 36), 61, 0.0, 2.0).cuda()
    calls = []
    real, real_tail = fused.conv_bn_lif, fused.lif_conv_bn_lif
    monkeypatch.setattr(fused, "conv_bn_lif", lambda *a, **k: calls.append(1) or real(*a, **k))
    monkeypatch.setattr(fused, "lif_conv_bn_lif", lambda *a, **k: calls.append(2) or real_tail(*a, **k))
    a = block(x)
    assert calls == [1, 2]   # the qkv chain with the contraction, then the attention neuron with the projection chain
    functional.reset_net(block)
    monkeypatch.setattr(fused, "conv_bn_lif", real)
    monkeypatch.setattr(fused, "lif_conv_bn_lif", real_tail)
    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", False)
    b = block(x)
    assert float((a != b).float().mean()) < 1e-3   # fp32 convolutions of two libraries: a spike in a thousand may flip


@pytest.mark.parametrize("where", ["proj_lif", "attn_lif", "qkv_lif", "proj_bn", "qkv_conv_pre", "qkv_container"])
def test_hooks_on_sub_modules_fire_and_see_the_spikes_of_the_unfused_path(where, monkeypatch):
    """A module with a hook is called the way the reference's forward calls it (layer/attention.py:370-384): the fused
    chain steps aside, the hook fires once per forward and sees what the same block computes with the fusion off."""
    block = _make_block(64, 2, 62).cuda().train()
    x = seeded_randn((4, 2, 64, 36), 63, 0.0, 2.0).cuda()
    seen = []
    target = {"proj_lif": block.proj_lif, "attn_lif": block.attn_lif, "qkv_lif": block.qkv_lif, "proj_bn": block.proj_conv_bn[1],
              "qkv_conv_pre": block.qkv_conv_bn[0], "qkv_container": block.qkv_conv_bn}[where]
    if where == "qkv_conv_pre":
        handle = target.register_forward_pre_hook(lambda m, args: seen.append(args[0].detach().clone()))
    else:
        handle = target.register_forward_hook(lambda m, args, out: seen.append(out.detach().clone()))
    out_hooked = block(x)
    assert len(seen) == 1
    handle.remove()
    functional.reset_net(block)
    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", False)
    handle = (target.register_forward_pre_hook(lambda m, args: seen.append(args[0].detach().clone())) if where == "qkv_conv_pre"
              else target.register_forward_hook(lambda m, args, out: seen.append(out.detach().clone())))
    out_plain = block(x)
    handle.remove()
    assert len(seen) == 2 and seen[0].shape == seen[1].shape
    if where in ("qkv_conv_pre", "qkv_container", "qkv_lif"):  # nothing fused ran in front of these: identical
        assert torch.equal(seen[0], seen[1])
    else:  # (a fused qkv chain ran in front of the hooked module: a spike in a thousand may differ, as between libraries)
        assert float((seen[0] != seen[1]).float().mean()) < 2e-3
    assert float((out_hooked != out_plain).float().mean()) < 2e-3


def test_autocast_keeps_the_modules_in_charge(monkeypatch):
    """Under autocast torch runs the convolution in the autocast dtype; the fused fp32 GEMMs would not, so they step aside."""
    from spikingjelly_amd.activation_based.layer import fused

    block = _make_block(64, 2, 64).cuda().train()
    x = seeded_randn((4, 2, 64, 36), 65, 0.0, 2.0).cuda()
    calls = []
    from spikingjelly_amd.activation_based.hip_kernel import conv_bn_lif as Ck
    monkeypatch.setattr(Ck, "conv_bn_lif_ssa", lambda *a, **k: calls.append(1))
    monkeypatch.setattr(Ck, "lif_conv_bn_lif", lambda *a, **k: calls.append(2))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = block(x)
    assert calls == [] and out.shape == x.shape


def test_cumulative_moving_average_batch_norm_runs_fused(monkeypatch):
    """``BatchNorm1d(momentum=None)``: the running statistics are the plain average over the batches seen, with the
    factor 1 / num_batches_tracked (nn.modules.batchnorm._BatchNorm.forward); the fused chain follows it step by step."""
    from spikingjelly_amd.activation_based.layer import fused

    fused_block, plain_block = _make_block(64, 2, 66).cuda().train(), _make_block(64, 2, 66).cuda().train()
    for block in (fused_block, plain_block):
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.momentum = None
    calls, real = [], fused.conv_bn_lif

    def recorded(*a, **k):
        r = real(*a, **k)
        if configure.hip_fuse_conv_bn_lif and a[1] is fused_block.qkv_conv_bn[0] and r is not None:
            calls.append(1)
        return r

    monkeypatch.setattr(fused, "conv_bn_lif", recorded)
    for step in range(3):
        x = seeded_randn((4, 2, 64, 36), 67 + step, 0.1 * step, 1.0 + step).cuda()
        monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", True)
        fused_block(x)
        monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", False)
        plain_block(x)
        functional.reset_net(fused_block)
        functional.reset_net(plain_block)
        for a, b in zip((fused_block.qkv_conv_bn[1], fused_block.proj_conv_bn[1]), (plain_block.qkv_conv_bn[1], plain_block.proj_conv_bn[1])):
            assert int(a.num_batches_tracked) == int(b.num_batches_tracked) == step + 1
            torch.testing.assert_close(a.running_mean, b.running_mean, rtol=1e-4, atol=1e-5)
            torch.testing.assert_close(a.running_var, b.running_var, rtol=1e-4, atol=1e-5)
    assert len(calls) == 3   # the fused block's qkv chain ran fused in every step


def test_sequences_longer_than_one_piece_stay_fused(monkeypatch):
    """T = 20 with gradients: the chain's backward walks the sequence in pieces of 16 steps, so the block keeps its
    fused path (the float64 comparison of this shape is a case of ``test_attention_block_fused_against_float64``)."""
    from spikingjelly_amd.activation_based.layer import fused

    block = _make_block(32, 2, 91).cuda().train()
    results, real = [], fused.conv_bn_lif

    def recorded(*a, **k):
        r = real(*a, **k)
        results.append(r is not None)
        return r

    monkeypatch.setattr(fused, "conv_bn_lif", recorded)
    x = seeded_randn((20, 2, 32, 36), 92, 0.0, 2.0).cuda().requires_grad_()
    block(x).sum().backward()
    assert results and results[0] and x.grad is not None and bool(torch.isfinite(x.grad).all())


def test_eval_mode_spikes_are_bit_identical_to_the_torch_backend_on_exact_inputs():
    """Binary input, weights that are multiples of 1/64, batch norm in evaluation mode with an exactly representable map
    (running variance + eps exactly 1, gamma and beta multiples of 1/8): every convolution sum and every normalised value is
    exact in fp32 in any order, so the hip block must fire exactly the spikes of the torch-backend block on the CPU."""
    torch.manual_seed(70)
    dim, heads, T, B, tokens = 64, 2, 4, 2, 36
    ref = layer.SpikingSelfAttention(dim, heads, backend="torch")
    g = torch.Generator().manual_seed(71)
    with torch.no_grad():
        for seq in (ref.qkv_conv_bn, ref.proj_conv_bn):
            seq[0].weight.copy_(torch.randint(-16, 17, seq[0].weight.shape, generator=g).float() / 64.0)
            seq[1].eps = 2.0 ** -10
            seq[1].running_var.fill_(1.0 - 2.0 ** -10)   # variance + eps is exactly 1
            seq[1].running_mean.copy_(torch.randint(-4, 5, (seq[1].num_features,), generator=g).float() / 8.0)
            seq[1].weight.copy_(torch.randint(4, 13, (seq[1].num_features,), generator=g).float() / 8.0)
            seq[1].bias.copy_(torch.randint(0, 9, (seq[1].num_features,), generator=g).float() / 8.0)
    ref.eval()
    hip = layer.SpikingSelfAttention(dim, heads, backend="hip")
    hip.load_state_dict(ref.state_dict())
    for a, b in ((hip.qkv_conv_bn, ref.qkv_conv_bn), (hip.proj_conv_bn, ref.proj_conv_bn)):
        a[1].eps = b[1].eps
    hip = hip.cuda().eval()
    x = (torch.rand((T, B, dim, tokens), generator=g) < 0.4).float()
    with torch.no_grad():
        want = ref(x)
        got = hip(x.cuda())
    assert torch.equal(got.cpu(), want)
    assert 0.02 < float(want.mean()) < 0.9


def test_pointwise_conv2d_bn_lif_module():
    from spikingjelly_amd.activation_based.model import spikformer

    torch.manual_seed(80)
    m = spikformer.SpikformerConv2dBNLIF(12, 20, kernel_size=1, backend="hip").cuda().train()
    x = seeded_randn((4, 2, 12, 6, 6), 81, 0.0, 2.0)
    ref = co.conv_bn_lif(x.double().flatten(3), m.conv_bn.block[0].weight.detach().double().cpu()[:, :, 0, 0],
                         m.conv_bn.block[1].weight.detach().double().cpu(), m.conv_bn.block[1].bias.detach().double().cpu(),
                         torch.zeros(20, dtype=torch.float64), torch.ones(20, dtype=torch.float64), True,
                         torch.zeros((2, 20, 36), dtype=torch.float64))
    assert _no_borderline(ref["h_seq"], 1.0)
    out = m(x.cuda())
    assert out.shape == (4, 2, 20, 6, 6)
    assert torch.equal(out.cpu().double().flatten(3), ref["spike_seq"])


@pytest.mark.parametrize("pool", [False, True])
def test_conv2d_3x3_bn_lif_module_against_float64_torch_modules(pool):
    """A 3x3 convolution stays with torch; batch norm and the neuron run fused when nothing sits between them."""
    from spikingjelly_amd.activation_based.model import spikformer

    torch.manual_seed(90)
    m = spikformer.SpikformerConv2dBNLIF(6, 8, kernel_size=3, stride=1, padding=1, pool=pool, backend="hip")
    ref = spikformer.SpikformerConv2dBNLIF(6, 8, kernel_size=3, stride=1, padding=1, pool=pool, backend="torch").double()
    ref.load_state_dict({k: v.double() if v.is_floating_point() else v for k, v in m.state_dict().items()})
    x = seeded_randn((4, 2, 6, 8, 8), 91, 0.0, 2.0)
    g = seeded_randn((4, 2, 8, 4, 4) if pool else (4, 2, 8, 8, 8), 92)
    x64 = x.double().requires_grad_()
    want = ref(x64)
    want.backward(g.double())
    m = m.cuda().train()
    xd = x.cuda().requires_grad_()
    out = m(xd)
    out.backward(g.cuda())
    assert float((out.detach().cpu().double() != want.detach()).float().mean()) == 0.0
    torch.testing.assert_close(xd.grad.cpu().double(), x64.grad, rtol=1e-3, atol=2e-5 * float(x64.grad.abs().max()))
    torch.testing.assert_close(m.conv_bn.block[0].weight.grad.cpu().double(), ref.conv_bn.block[0].weight.grad, rtol=1e-3,
                               atol=2e-5 * float(ref.conv_bn.block[0].weight.grad.abs().max()))
