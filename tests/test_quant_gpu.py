"""GPU parity: lightcompress_amd quantizers / packers vs the CPU oracle, bit-exact."""
import pytest
import torch

from oracle import pack_ref, quant_ref as Q
from tests.helpers import assert_bit_equal, gen, weight_like

pytestmark = pytest.mark.gpu


def _iq(bit, sym, gran, **kw):
    from lightcompress_amd import IntegerQuantizer
    return IntegerQuantizer(bit, sym, gran, **kw)


INT_CASES = [
    # bit, sym, granularity, kwargs, shape
    (4, False, 'per_group', dict(group_size=128), (256, 1024)),
    (4, True, 'per_group', dict(group_size=128), (256, 1024)),
    (4, False, 'per_group', dict(group_size=64), (128, 512)),
    (4, False, 'per_group', dict(group_size=32), (128, 256)),
    (3, False, 'per_group', dict(group_size=256), (64, 1024)),
    (8, True, 'per_channel', {}, (300, 4096)),
    (8, False, 'per_channel', {}, (64, 11008)),
    (4, False, 'per_channel', {}, (33, 1000)),       # 1000 % 8 == 0, % 16 != 0
    (8, True, 'per_channel', {}, (17, 1001)),        # odd length -> element-wise kernel
    (8, True, 'per_tensor', {}, (128, 512)),
    (8, False, 'per_tensor', {}, (128, 512)),
    (4, False, 'per_group', dict(group_size=128, round_zp=False), (64, 512)),
    (6, True, 'per_head', dict(head_num=8), (64, 512)),
]


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('bit,sym,gran,kw,shape', INT_CASES)
def test_int_fake_and_real_quant_bit_exact(dev, dtype, bit, sym, gran, kw, shape):
    w = weight_like(*shape, seed=bit + shape[0], dtype=dtype, outlier_frac=0.002)
    spec = Q.IntSpec(bit, sym, gran, group_size=kw.get('group_size', 0), head_num=kw.get('head_num', 0),
                     round_zp=kw.get('round_zp', True))
    q = _iq(bit, sym, gran, **kw)
    wd = w.to(dev)

    assert_bit_equal(q.fake_quant_weight_dynamic(wd), Q.int_fake_quant_dynamic(spec, w), 'fake_quant_weight_dynamic')

    rows, s, z, qmax, qmin = q.get_tensor_qparams(wd)
    orows, os_, oz, _, _ = Q.int_tensor_qparams(spec, w)
    assert tuple(rows.shape) == tuple(orows.shape)
    assert_bit_equal(s, os_, 'scales')
    if not sym:
        assert_bit_equal(z, oz, 'zeros')

    assert_bit_equal(q.quant(rows, s, z, qmax, qmin), Q.int_quant(spec, orows, os_, oz, spec.qmax, spec.qmin), 'quant')
    assert_bit_equal(q.quant_dequant(rows, s, z, qmax, qmin),
                     Q.int_quant_dequant(spec, orows, os_, oz, spec.qmax, spec.qmin), 'quant_dequant')

    if kw.get('round_zp', True) and gran != 'per_head':      # per_head real quant raises in the reference too
        codes, rs, rz = q.real_quant_weight_dynamic(wd)
        ocodes, ors, orz = Q.int_real_quant_dynamic(spec, w)
        assert_bit_equal(codes, ocodes, 'codes')
        assert_bit_equal(rs, ors, 'real scales')
        assert (rz is None) == (orz is None)
        if rz is not None:
            assert_bit_equal(rz, orz, 'real zeros')


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_int_static_paths_and_minmax(dev, dtype):
    w = weight_like(128, 1024, seed=21, dtype=dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    q = _iq(4, False, 'per_group', group_size=128)
    orows, os_, oz, oqmax, oqmin = Q.int_tensor_qparams(spec, w)
    # qparams from one tensor applied to another (static), with an output scale factor
    w2 = weight_like(128, 1024, seed=22, dtype=dtype)
    args = dict(scales=os_.to(dev), zeros=oz.to(dev), qmax=oqmax, qmin=oqmin, output_scale_factor=0.5)
    got = q.fake_quant_weight_static(w2.to(dev), dict(args))
    want = Q.int_fake_quant_static(spec, w2, os_, oz, oqmax, oqmin, output_scale_factor=0.5)
    assert_bit_equal(got, want, 'fake_quant_weight_static')
    codes, s, z = q.real_quant_weight_static(w2.to(dev), dict(args))
    ocodes, os2, oz2 = Q.int_real_quant_static(spec, w2, os_, oz, oqmax, oqmin, output_scale_factor=0.5)
    assert_bit_equal(codes, ocodes, 'static codes')
    assert_bit_equal(s, os2, 'static scales')
    assert_bit_equal(z, oz2, 'static zeros')
    mn, mx = q.get_minmax_range(q.reshape_tensor(w.to(dev)))
    omn, omx = Q.minmax_range(spec, orows)
    assert_bit_equal(mn, omn, 'min'); assert_bit_equal(mx, omx, 'max')
    s3, z3, _, _ = q.get_qparams((mn, mx), dev)
    assert_bit_equal(s3, os_, 'get_qparams scales'); assert_bit_equal(z3, oz, 'get_qparams zeros')
    dq = q.dequant(q.quant(q.reshape_tensor(w.to(dev)), s3, z3, oqmax, oqmin), s3, z3)
    assert_bit_equal(dq, Q.int_dequant(Q.int_quant(spec, orows, os_, oz, oqmax, oqmin), os_, oz), 'dequant')
    # activations: per-token rows of a 3-D tensor
    act = (torch.randn(4, 64, 512, generator=gen(23)) * 3).to(dtype)
    aq = _iq(8, True, 'per_token')
    assert_bit_equal(aq.fake_quant_act_dynamic(act.to(dev)), Q.int_fake_quant_dynamic(Q.IntSpec(8, True, 'per_token'), act), 'act')


def test_int_boundary_cases_hit_the_exact_division_path(dev):
    """Inputs built to sit on and next to rounding ties (k + 0.5) * s."""
    g = gen(31)
    s = (torch.rand(512, 1, generator=g) * 0.01 + 1e-3)
    k = torch.randint(0, 15, (512, 128), generator=g).float()
    ulp = torch.randint(-2, 3, (512, 128), generator=g)
    x = ((k + 0.5) * s)
    x = (x.view(torch.int32) + ulp).view(torch.float32)
    x[:, 0] = 0.0
    x[:, 1] = s[:, 0] * 15                                   # pins min = 0 and max = 15 * s
    for dtype in (torch.float32, torch.bfloat16):
        xd = x.to(dtype)
        spec = Q.IntSpec(4, False, 'per_group', group_size=128)
        got = _iq(4, False, 'per_group', group_size=128).real_quant_weight_dynamic(xd.to(dev))
        want = Q.int_real_quant_dynamic(spec, xd)
        assert_bit_equal(got[0], want[0], f'tie codes {dtype}')
        assert_bit_equal(got[1], want[1], f'tie scales {dtype}')


def test_int_edge_shapes(dev):
    q = _iq(4, False, 'per_group', group_size=128)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    # fewer columns than a group: one row-wise range (quant.py:613-631)
    w = weight_like(8, 96, seed=41)
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.int_fake_quant_dynamic(spec, w), 'short rows')
    # constant rows: the 1e-5 clamp decides the scale
    w = torch.full((4, 128), 0.25)
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.int_fake_quant_dynamic(spec, w), 'constant rows')
    w = torch.zeros(4, 128, dtype=torch.bfloat16)
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.int_fake_quant_dynamic(spec, w), 'zero rows')
    # a single group, and a row count that does not fill a wave
    w = weight_like(1, 128, seed=42)
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.int_fake_quant_dynamic(spec, w), 'one group')
    w = weight_like(3, 640, seed=43, dtype=torch.bfloat16)
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.int_fake_quant_dynamic(spec, w), 'ragged')
    # transposed view ('dim': 'ic')
    w = weight_like(256, 64, seed=44)
    got = q.fake_quant_weight_dynamic(w.to(dev), {'dim': 'ic'})
    want = Q.int_fake_quant_dynamic(spec, w.T).T
    assert_bit_equal(got.contiguous(), want.contiguous(), 'dim=ic')


FP_CASES = [('e4m3', 'per_channel', (64, 7168)), ('e4m3', 'per_channel', (128, 2048)), ('e4m3', 'per_token', (96, 7168)),
            ('e5m2', 'per_channel', (64, 1024)), ('e4m3', 'per_group', (64, 1024)), ('e4m3', 'per_tensor', (64, 512)),
            ('e2m1', 'per_group', (64, 512)), ('e3m2', 'per_channel', (32, 520)), ('e4m3', 'per_channel', (9, 1003))]


@pytest.mark.parametrize('tie', ['away', 'even'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fmt,gran,shape', FP_CASES)
def test_float_quant_bit_exact(dev, tie, dtype, fmt, gran, shape):
    from lightcompress_amd import FloatQuantizer
    w = weight_like(*shape, seed=shape[1], dtype=dtype, std=0.006, outlier_frac=0.0005, outlier_mul=30)
    w[0, :4] = torch.tensor([0.0, -0.0, 1e-9, -1e-9], dtype=dtype)      # zeros and deep subnormal-range values
    kw = dict(group_size=128) if gran == 'per_group' else {}
    spec = Q.FloatSpec(fmt, gran, group_size=kw.get('group_size', 0), tie=tie)
    q = FloatQuantizer(fmt, True, gran, use_qtorch=True, fp_tie=tie, **kw)
    wd = w.to(dev)
    assert_bit_equal(q.fake_quant_weight_dynamic(wd), Q.float_fake_quant_dynamic(spec, w), 'float fake quant')
    rows, s, z, qmax, qmin = q.get_tensor_qparams(wd)
    orows, os_, oz, _, _ = Q.float_tensor_qparams(spec, w)
    assert_bit_equal(s, os_, 'float scales')
    assert_bit_equal(q.quant(rows, s.clone(), z, qmax, qmin), Q.float_quant(spec, orows, os_.clone(), oz), 'float quant')
    want_dq = Q.float_dequant(Q.float_quant(spec, orows, os_.clone(), oz), os_, oz)
    assert_bit_equal(q.quant_dequant(rows, s.clone(), z, qmax, qmin), want_dq, 'float quant_dequant')
    if fmt in ('e4m3', 'e5m2'):
        codes, rs, rz = q.real_quant_weight_dynamic(wd)
        ocodes, ors, _ = Q.float_real_quant_dynamic(spec, w)
        assert rz is None
        assert_bit_equal(codes, ocodes, 'fp8 codes')
        assert_bit_equal(rs, ors, 'fp8 scales')


@pytest.mark.parametrize('tie', ['away', 'even'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fmt,top', [('e4m3', 448.0), ('e5m2', 57344.0)])
def test_float_quant_given_scales_around_the_float8_maximum(dev, tie, dtype, fmt, top):
    """Given scales let quotients pass the float8 maximum, where the reference's grid goes on (480 after 448, 65536
    after 57344) and a hardware float8 convert would saturate: every bf16 number of magnitude 0.8 .. 1.25 times the
    maximum, divided by scales that put the quotients between bf16 numbers (a bf16 row rounds them again)."""
    from lightcompress_amd import FloatQuantizer
    base = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    base = base[torch.isfinite(base) & (base.abs() >= 0.8 * top) & (base.abs() <= 1.25 * top)]
    base = base[: base.numel() // 8 * 8]
    factors = [1.0, 1.0234375, 0.98828125, 1.0078125, 1.046875, 0.9609375]
    x = base[None, :].repeat(len(factors), 1).to(dtype)
    spec = Q.FloatSpec(fmt, 'per_channel', tie=tie)
    q = FloatQuantizer(fmt, True, 'per_channel', use_qtorch=True, fp_tie=tie)
    rows, s, z, qmax, qmin = q.get_tensor_qparams(x.to(dev))
    orows, os_, oz, _, _ = Q.float_tensor_qparams(spec, x)
    mine = torch.tensor(factors, dtype=dtype).reshape(-1, 1)
    want = Q.float_quant(spec, orows, mine.clone(), oz)
    assert float(want.abs().max()) > top                    # the case is there: codes beyond the float8 maximum
    assert_bit_equal(q.quant(rows, mine.to(dev), z, qmax, qmin), want, 'float quant, given scales')
    assert_bit_equal(q.quant_dequant(rows, mine.to(dev), z, qmax, qmin),
                     Q.float_dequant(Q.float_quant(spec, orows, mine.clone(), oz), mine, oz), 'float quant_dequant, given scales')


def _agree(a, b):
    return float((a.cpu().float() == b.float()).float().mean())


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fmt,gran,shape', [('e4m3', 'per_channel', (64, 2048)), ('e4m3', 'per_group', (64, 1024)),
                                            ('e5m2', 'per_channel', (32, 1024)), ('e2m1', 'per_group', (64, 512)),
                                            ('e4m3', 'per_token', (96, 7168))])
def test_float_emulation_without_qtorch(dev, dtype, fmt, gran, shape):
    """use_qtorch=False (quant.py:1004-1026): scales 2 ** (floor(log2|x| + bias) - m - bias) per element.  The kernel
    takes log2 and 2 ** x from the functions torch's GPU kernels use, so it is compared bit for bit with the oracle
    evaluated on GPU tensors, which is the reference's own evaluation.  bf16 rows round every intermediate to 8 bits,
    which hides the last place of the math library: they also equal the oracle on CPU tensors bit for bit.  fp32 rows
    on the CPU come from another math library (the last place of a row's bias moves every scale of the row by 1.3e-6):
    there the results agree to 4e-6 relative."""
    from lightcompress_amd import FloatQuantizer
    kw = dict(group_size=128) if gran == 'per_group' else {}
    spec = Q.FloatSpec(fmt, gran, group_size=kw.get('group_size', 0))
    q = FloatQuantizer(fmt, True, gran, use_qtorch=False, **kw)
    for case in range(2):
        if case == 0:
            w = weight_like(*shape, seed=shape[1] + 1, dtype=dtype, std=0.006, outlier_frac=0.0005, outlier_mul=30)
        else:                                               # row maxima of every size: the bias takes many values
            w = (torch.randn(*shape, generator=gen(shape[1] + 2)) * 0.05 * torch.exp(torch.randn(shape[0], 1, generator=gen(3)))).to(dtype)
        w[0, :2] = torch.tensor([0.0, -0.0], dtype=dtype)
        wd = w.to(dev)
        got = q.fake_quant_weight_dynamic(wd)
        on_gpu = Q.float_emu_fake_quant_dynamic(spec, wd.clone())
        assert_bit_equal(got, on_gpu, f'fake quant against the oracle on GPU tensors (case {case})')
        on_cpu = Q.float_emu_fake_quant_dynamic(spec, w.clone())
        if dtype == torch.bfloat16:
            assert_bit_equal(got, on_cpu, f'fake quant against the oracle on CPU tensors (case {case})')
        elif dtype == torch.float16:                       # 11-bit intermediates: the math library shows now and then
            assert _agree(got, on_cpu) >= 0.99
        else:
            near = (got.cpu().double() - on_cpu.double()).abs() <= on_cpu.double().abs() * 4e-6 + 1e-30
            assert float(near.float().mean()) >= 0.999
        xc, s, z, qmax, qmin = q.get_tensor_qparams(wd)
        oxc, os_, oz, _, _ = Q.float_emu_tensor_qparams(spec, wd.clone())
        assert qmax is None and qmin is None and z.dtype == torch.int64 and int(z) == 0
        assert_bit_equal(xc, oxc, 'clamped tensor')
        assert_bit_equal(s, os_, 'scales')
        assert_bit_equal(q.quant(xc, s.clone(), z, None, None), Q.float_emu_quant(oxc, os_.clone(), oz), 'round(t / s)')
        oq = Q.float_emu_quant(oxc, os_.clone(), oz)
        assert_bit_equal(q.dequant(oq, os_, z), Q.float_dequant(oq, os_, oz), 'q * s')
        assert_bit_equal(q.quant_dequant(xc, os_.clone(), z, None, None), Q.float_dequant(oq, os_, oz), 'quant_dequant')
        assert_bit_equal(q.fake_quant_weight_static(wd, dict(scales=os_.clone(), zeros=z, qmax=None, qmin=None)),
                         Q.restore_rows(spec, Q.float_dequant(oq, os_, oz), w.shape).to(dtype), 'static fake quant')
        if fmt in ('e4m3', 'e5m2') and gran == 'per_channel':
            codes, rs, rz = q.real_quant_weight_dynamic(wd)
            ocodes, ors, _ = Q.float_emu_real_quant_dynamic(spec, wd.clone())
            assert rz is None
            assert_bit_equal(codes, ocodes, 'float8 codes')
            assert_bit_equal(rs, ors, 'elementwise scales')


def test_float_emulation_per_tensor_raises_like_the_reference(dev):
    from lightcompress_amd import FloatQuantizer
    q = FloatQuantizer('e4m3', True, 'per_tensor', use_qtorch=False)
    with pytest.raises(IndexError):                 # maxval.shape[0] of a 0-dim range, quant.py:1011
        q.fake_quant_weight_dynamic(weight_like(8, 64, seed=5).to(dev))


def test_float_act_fake_quant_3d(dev):
    from lightcompress_amd import FloatQuantizer
    act = (torch.randn(2, 48, 7168, generator=gen(51)) * torch.exp(torch.randn(7168, generator=gen(52)))).bfloat16()
    q = FloatQuantizer('e4m3', True, 'per_token', use_qtorch=True)
    assert_bit_equal(q.fake_quant_act_dynamic(act.to(dev)), Q.float_fake_quant_dynamic(Q.FloatSpec('e4m3', 'per_token'), act), 'fp8 act')


@pytest.mark.parametrize('bits,dt', [(4, torch.int32), (8, torch.int8)])
@pytest.mark.parametrize('shape', [(64, 4096), (7, 37), (128, 7168), (3, 8)])
def test_pack_ct_bit_exact(dev, bits, dt, shape):
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    lo = -(1 << (bits - 1))
    codes = torch.randint(lo, -lo, shape, generator=gen(61), dtype=dt)
    scales = torch.rand(shape[0], 1, generator=gen(62))
    got, gs = VllmRealQuantLinear.pack(codes.to(dev), scales.to(dev), {'weight': {'bit': bits}})
    want, ws = pack_ref.pack_ct(codes, scales, bits)
    assert_bit_equal(got, want, 'packed'); assert_bit_equal(gs, ws, 'fp16 scales')
    assert torch.equal(pack_ref.unpack_ct(got.cpu(), bits, shape[1]), codes.to(torch.int32))


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize('gran,shape', [('per_group', (64, 1024)), ('per_group', (2048, 7168)), ('per_channel', (96, 512)),
                                        ('per_channel', (16, 7168))])
def test_fused_quant_pack_equals_quant_then_pack(dev, dtype, gran, shape):
    """One-pass quantize+pack == VllmRealQuantLinear.pack(real_quant_weight_dynamic(w)) == the oracle's pack."""
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    w = weight_like(*shape, seed=shape[1] + 7, dtype=dtype, std=0.006, outlier_frac=0.0005, outlier_mul=30)
    kw = dict(group_size=128) if gran == 'per_group' else {}
    q = IntegerQuantizer(4, True, gran, **kw)
    cfg = {'weight': {'bit': 4}}
    wd = w.to(dev)
    codes, s, z = q.real_quant_weight_dynamic(wd)
    two_step, s16 = VllmRealQuantLinear.pack(codes, s, cfg)
    fused, fs16 = VllmRealQuantLinear.quant_pack_fused(wd, q, cfg)
    assert_bit_equal(fused, two_step, 'packed words')
    assert_bit_equal(fs16, s16, 'fp16 scales')
    spec = Q.IntSpec(4, True, gran, group_size=kw.get('group_size', 0))
    ocodes, os_, _ = Q.int_real_quant_dynamic(spec, w)
    opacked, _ = pack_ref.pack_ct(ocodes, os_, 4)
    assert_bit_equal(fused, opacked, 'oracle pack')


@pytest.mark.parametrize('scale', [1.0, 0.5, 0.015625, 4.0])
def test_fused_quant_pack_on_rounding_ties_and_clamp_bounds(dev, scale):
    """The one-pass bf16 quantize + pack takes its nibbles from the biased quotient (t + 1.5 * 2^23): every half-integer
    quotient (ties go to the even code), both clamp bounds, zeros of both signs, and values just beside the ties."""
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    halves = torch.arange(-19, 20, dtype=torch.float32) * 0.5            # -9.5 .. 9.5 in steps of 0.5
    near = torch.cat([halves + 0.0625, halves - 0.0625])
    vals = torch.cat([halves, near, torch.tensor([0.0, -0.0, 7.0, -7.0, -8.0, 6.9375])])
    vals = vals[vals.abs() <= 7.0]                                        # the row maximum fixes the scale: 7 * scale / 7
    row = torch.zeros(128)
    row[:vals.numel()] = vals
    row[-1] = 7.0
    w = (torch.stack([row, -row, row.flip(0), row * 0.5]) * scale).bfloat16()
    assert torch.equal(w[0].float(), row * scale)                         # every value is a bf16 number
    q = IntegerQuantizer(4, True, 'per_group', group_size=128)
    spec = Q.IntSpec(4, True, 'per_group', group_size=128)
    fused, fs16 = VllmRealQuantLinear.quant_pack_fused(w.to(dev), q, {'weight': {'bit': 4}})
    ocodes, os_, _ = Q.int_real_quant_dynamic(spec, w)
    assert float(os_[0]) == scale and int(ocodes.min()) >= -8 and int(ocodes.max()) == 7
    opacked, _ = pack_ref.pack_ct(ocodes, os_, 4)
    assert_bit_equal(fused, opacked, 'packed words on ties')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('shape', [(64, 256), (320, 1024), (2048, 512)])
def test_gemm_pack_bit_exact(dev, dtype, shape):
    from lightcompress_amd.module_utils import AutoawqRealQuantLinear
    w = weight_like(*shape, seed=71, dtype=dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    _, s, z = Q.int_real_quant_dynamic(spec, w.float() if dtype == torch.float16 else w)
    s = s.to(dtype)
    cfg = {'weight': {'bit': 4, 'group_size': 128}}
    got = AutoawqRealQuantLinear.gemm_pack(None, w.to(dev), s.to(dev), z.to(dev), cfg)
    want = pack_ref.gemm_pack(w, s, z, 128)
    for a, b, n in zip(got, want, ('qweight', 'scales', 'qzeros')):
        assert_bit_equal(a, b, n)


def test_full_size_rtn_properties(dev):
    """BASELINE config 1 at full size, through size-independent properties."""
    w = weight_like(4096, 4096, seed=0)
    q = _iq(4, False, 'per_group', group_size=128)
    wd = w.to(dev)
    codes, s, z = q.real_quant_weight_dynamic(wd)
    fq = q.fake_quant_weight_dynamic(wd)
    assert codes.dtype == torch.int32 and int(codes.min()) == 0 and int(codes.max()) == 15
    # dequantising the codes reproduces the fake-quantised weights exactly
    dq = ((codes.view(-1, 128).float() - z.view(-1, 1).float()) * s.view(-1, 1)).view(4096, 4096)
    assert torch.equal(dq, fq)
    assert float((fq - wd).abs().max()) <= float(s.max()) * 0.5001
    # idempotence: fake-quantising the result again is a fixed point of the codes
    codes2, _, _ = q.real_quant_weight_static(fq, {'scales': s.view(-1, 1), 'zeros': z.view(-1, 1).float(), 'qmax': q.qmax, 'qmin': q.qmin})
    assert torch.equal(codes2, codes)
    # a 256-row slice against the oracle, bit for bit
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    oc, os_, oz = Q.int_real_quant_dynamic(spec, w[1000:1256])
    assert_bit_equal(codes[1000:1256], oc, 'slice codes'); assert_bit_equal(s[1000:1256], os_, 'slice scales')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize('shape', [(256, 384), (200, 296), (2048, 7168), (129, 8)])
def test_blockwise_fp8_casts_bit_exact(dev, dtype, shape):
    """kernel.py (Triton semantics) and the FloatQuantizer per_block route, against their oracles: codes, scales and
    the dequantized weight bit for bit."""
    from lightcompress_amd import kernel as K8, FloatQuantizer
    from lightcompress_amd.quant import weight_cast_to_bf16 as q_to_bf16, weight_cast_to_fp8 as q_to_fp8
    w = weight_like(*shape, seed=shape[1] + 3, dtype=dtype, std=0.006, outlier_frac=0.0005, outlier_mul=30)
    w[0, :4] = torch.tensor([0.0, -0.0, 1e-9, -1e-9], dtype=dtype)
    wd = w.to(dev)
    y, s = K8.weight_cast_to_fp8(wd)
    oy, os_ = Q.triton_weight_cast_to_fp8(w)
    assert y.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == os_.shape
    assert_bit_equal(s, os_, 'block scales')
    assert_bit_equal(y.view(torch.uint8), oy.view(torch.uint8), 'fp8 codes')
    torch.set_default_dtype(torch.bfloat16)
    try:
        back = K8.weight_cast_to_bf16(y, s)
    finally:
        torch.set_default_dtype(torch.float32)
    assert_bit_equal(back, Q.triton_weight_cast_to_bf16(oy, os_), 'block dequant')
    assert_bit_equal(q_to_bf16(y, s, 128), Q.triton_weight_cast_to_bf16(oy, os_), 'quant.py weight_cast_to_bf16')
    for tie in ('away', 'even'):
        fq = FloatQuantizer('e4m3', True, 'per_block', block_size=128, use_qtorch=True, fp_tie=tie)
        yq, sq, zq = fq.real_quant_weight_dynamic(wd)
        oyq, osq, _ = Q.float_per_block_real_quant(Q.FloatSpec('e4m3', 'per_block', tie=tie), w)
        assert zq is None
        assert_bit_equal(sq, osq, 'per_block scales')
        assert_bit_equal(yq.view(torch.uint8), oyq.view(torch.uint8), f'per_block codes tie={tie}')
    # reshape_tensor / restore_tensor for per_block (quant.py:634-651): zero-padded block view and back
    fq = FloatQuantizer('e4m3', True, 'per_block', block_size=128, use_qtorch=True)
    blocks = fq.reshape_tensor(wd)
    mp, np_ = -(-shape[0] // 128) * 128, -(-shape[1] // 128) * 128
    assert blocks.shape == (mp // 128, 128, np_ // 128, 128)
    pad = torch.zeros(mp, np_, dtype=w.dtype)
    pad[:shape[0], :shape[1]] = w
    assert torch.equal(blocks.cpu(), pad.view(-1, 128, np_ // 128, 128))
    if shape[1] % 128 == 0:
        assert torch.equal(fq.restore_tensor(blocks, wd.shape).cpu(), w)
    # (with padded columns the reference's restore either raises or returns rows of the padded matrix: not a use case)
    y2, s2 = q_to_fp8(wd, 128)
    oy2, os2, _ = Q.float_per_block_real_quant(Q.FloatSpec('e4m3', 'per_block'), w)
    assert_bit_equal(y2.view(torch.uint8), oy2.view(torch.uint8), 'quant.py weight_cast_to_fp8')
    if shape[1] % 128 == 0:
        ya, sa = K8.act_quant(wd)
        oya, osa = Q.triton_act_quant(w)
        assert_bit_equal(sa, osa, 'act scales')
        assert_bit_equal(ya.view(torch.uint8), oya.view(torch.uint8), 'act codes')


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fmt,gran,shape,tie', [('e4m3', 'per_channel', (48, 1024), 'away'), ('e4m3', 'per_group', (16, 512), 'even'),
                                                ('e2m1', 'per_group', (32, 256), 'away')])
def test_float_quantizer_with_mse_and_learnable_ranges(dev, dtype, fmt, gran, shape, tie):
    """FloatQuantizer with calib_algo 'mse' / 'learnable' (the range dispatch of quant.py:124-132 is shared by both
    quantizer classes).  The mse search sums |d|**2.4 through another pow and another summation order than the CPU's,
    so a step that ties with the running best within ~1e-6 may be accepted on one side only: the ranges agree on
    >= 98 % of the rows, the others are as good within 0.1 %; given the ranges, fake and real quantization are the
    bit-exact static path."""
    from lightcompress_amd import FloatQuantizer
    kw = dict(group_size=128) if gran == 'per_group' else {}
    w = weight_like(*shape, seed=shape[1] + 3, dtype=dtype, std=0.006, outlier_frac=0.002, outlier_mul=30)
    spec = Q.FloatSpec(fmt, gran, group_size=kw.get('group_size', 0), tie=tie)
    q = FloatQuantizer(fmt, True, gran, use_qtorch=True, fp_tie=tie, calib_algo='mse', **kw)
    rows = Q.reshape_rows(spec, w)
    omn, omx = Q.float_mse_range(spec, rows.clone())
    mn, mx = q.get_mse_range(q.reshape_tensor(w.to(dev)))
    assert mn.dtype == torch.float32 and mn.shape == omn.shape
    same = ((mn.cpu() - omn).abs() <= 1e-6 * omn.abs()) & ((mx.cpu() - omx).abs() <= 1e-6 * omx.abs())
    assert float(same.float().mean()) >= 0.98, float(same.float().mean())
    def err(lo, hi):
        s, z, _, _ = Q.float_qparams(spec, lo, hi)
        return (Q.float_dequant(Q.float_quant(spec, rows.float(), s, z), s, z) - rows.float()).abs().pow(2.4).sum(1)
    assert bool((err(mn.cpu(), mx.cpu()) <= err(omn, omx) * 1.001 + 1e-30).all())
    got = q.fake_quant_weight_dynamic(w.to(dev))
    assert got.dtype == dtype
    assert_bit_equal(got, Q.float_fake_quant_with_range(spec, w, mn.cpu(), mx.cpu()), 'fake quant with the mse ranges')
    if fmt == 'e4m3':
        codes, s, z = q.real_quant_weight_dynamic(w.to(dev))
        os_, oz, _, _ = Q.float_qparams(spec, mn.cpu(), mx.cpu())
        assert z is None and codes.dtype == torch.float8_e4m3fn
        assert_bit_equal(codes, Q.restore_rows(spec, Q.float_quant(spec, rows, os_.clone(), oz), w.shape).to(torch.float8_e4m3fn), 'fp8 codes')
        assert_bit_equal(s, os_.view(w.shape[0], -1), 'fp8 scales')
    # learnable: the given factors scale the symmetric range, everything after is the static path
    ql = FloatQuantizer(fmt, True, gran, use_qtorch=True, fp_tie=tie, calib_algo='learnable', **kw)
    # factors whose sigmoid is the same number whatever library evaluates it: sigmoid(0) = 1/2, sigmoid(20) rounds to 1
    up = torch.where(torch.rand(rows.shape[0], 1, generator=gen(7)) < 0.5, 0.0, 20.0).to(dtype)
    lo, hi = Q.learnable_range(spec, rows, upbound_factor=up)
    got = ql.fake_quant_weight_dynamic(w.to(dev), {'upbound_factor': up.to(dev)})
    assert_bit_equal(got, Q.float_fake_quant_with_range(spec, w, lo, hi), 'fake quant with learnable ranges')
    assert_bit_equal(ql.fake_quant_weight_dynamic(w.to(dev)), Q.float_fake_quant_dynamic(spec, w), 'learnable without factors')
    with pytest.raises(NotImplementedError):
        FloatQuantizer(fmt, True, gran, use_qtorch=True, calib_algo='hqq', **kw).fake_quant_weight_dynamic(w.to(dev))


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('bit,sym,gran,shape', [(4, False, 'per_group', (64, 1024)), (4, True, 'per_group', (32, 512)),
                                                 (8, False, 'per_channel', (48, 777)), (3, False, 'per_group', (16, 256))])
def test_mse_calibration_against_oracle(dev, dtype, bit, sym, gran, shape):
    """calib_algo='mse' (quant.py:147-205).  |d|**2.4 goes through powf and the row sum through another summation
    order than torch's, so a step whose error ties with the running best within ~1e-6 may be accepted on one side
    only: the found ranges agree on >= 99 % of the rows, and on the others the |.|^2.4 error of the kernel's range
    is within 0.1 % of the oracle's.  Given the same ranges everything downstream is the bit-exact static path."""
    from lightcompress_amd import IntegerQuantizer
    kw = dict(group_size=128) if gran == 'per_group' else {}
    w = weight_like(*shape, seed=shape[1] + bit, dtype=dtype)
    spec = Q.IntSpec(bit, sym, gran, group_size=kw.get('group_size', 0))
    q = IntegerQuantizer(bit, sym, gran, calib_algo='mse', **kw)
    rows = Q.reshape_rows(spec, w)
    omn, omx = Q.int_mse_range(spec, rows.clone())
    mn, mx = q.get_mse_range(q.reshape_tensor(w.to(dev)))
    assert mn.dtype == torch.float32 and mn.shape == omn.shape
    same = ((mn.cpu() - omn).abs() <= 1e-6 * omn.abs()) & ((mx.cpu() - omx).abs() <= 1e-6 * omx.abs())
    assert float(same.float().mean()) >= 0.99
    def err(lo, hi):
        s, z, qmax, qmin = Q.int_qparams(spec, lo, hi)
        return (Q.int_quant_dequant(spec, rows.float(), s, z, qmax, qmin) - rows.float()).abs().pow(2.4).sum(1)
    e_k, e_o = err(mn.cpu(), mx.cpu()), err(omn, omx)
    assert bool((e_k <= e_o * 1.001 + 1e-30).all())
    # end to end through the calibrated static path
    got = q.fake_quant_weight_dynamic(w.to(dev))
    s, z, qmax, qmin = Q.int_qparams(spec, mn.cpu(), mx.cpu())
    want = Q.restore_rows(spec, Q.int_quant_dequant(spec, rows, s, z, qmax, qmin), w.shape).to(dtype)
    assert_bit_equal(got, want, 'fake quant with the calibrated ranges')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('bit,sym,gran,kw,shape,hqq', [
    (4, False, 'per_group', dict(group_size=64), (64, 512), {}),
    (4, False, 'per_group', dict(group_size=128), (32, 1024), dict(lp_norm=1, beta=20)),
    (3, False, 'per_channel', {}, (24, 1000), dict(iters=5)),
    (4, True, 'per_channel', {}, (16, 768), {}),
])
def test_hqq_calibration_against_oracle(dev, dtype, bit, sym, gran, kw, shape, hqq):
    """calib_algo='hqq' (quant.py:587-609, 679-687).  The scales are 1/(1/s), bit for bit.  The zero points are row
    means of fp32 terms that go through powf: they agree to 1e-5 absolute (they are of the order of qmax: a few ulp,
    from the order of the row sums; the oracle evaluated on GPU tensors is as far away), the
    solver stops after the same number of iterations, and fake quantization with the kernel's own (scales, zeros)
    is the bit-exact static path."""
    from lightcompress_amd import IntegerQuantizer
    w = weight_like(*shape, seed=shape[1] + bit, dtype=dtype)
    spec = Q.IntSpec(bit, sym, gran, group_size=kw.get('group_size', 0))
    q = IntegerQuantizer(bit, sym, gran, calib_algo='hqq', **kw, **hqq)
    rows = Q.reshape_rows(spec, w.float())
    lo, hi = Q.minmax_range(spec, rows)
    s0, z0, qmax, qmin = Q.int_qparams(spec, lo, hi)
    os_, oz, n_ref = Q.hqq_optimize(rows, s0, z0, qmax, qmin, **hqq)
    t, s, z, _, _ = q.get_tensor_qparams(w.to(dev))
    assert t.dtype == torch.float32 and s.shape == os_.shape and z.shape == oz.shape
    assert_bit_equal(s, os_, 'hqq scales')
    assert float((z.cpu() - oz).abs().max()) <= 1e-5
    # same stopping point: one more iteration from the oracle's result would not be accepted either way; compare
    # the iteration count through the solver's own bookkeeping
    calls = []
    orig = q.optimize_weights_proximal
    import lightcompress_amd._lib as L
    real = L.lib().lcq_hqq_step
    class Counting:
        def __call__(self, *a):
            calls.append(1)
            return real(*a)
    L.lib().lcq_hqq_step = Counting()
    try:
        orig(t, s0.to(dev), z0 if sym else z0.to(dev), qmax, qmin)
    finally:
        L.lib().lcq_hqq_step = real
    assert len(calls) == n_ref
    got = q.fake_quant_weight_dynamic(w.to(dev))
    want = Q.restore_rows(spec, Q.int_quant_dequant(spec, rows, s.cpu(), z.cpu(), qmax, qmin), w.shape).to(w.dtype)
    assert_bit_equal(got, want, 'fake quant with the refined zero points')


def test_static_activation_calibration(dev):
    """static_minmax / static_moving_minmax (quant.py:252-262, 523-585): ranges bit-equal to the oracle's, qparams
    through get_qparams, one entry per module input."""
    from lightcompress_amd import IntegerQuantizer
    g = gen(11)
    acts = [torch.randn(4, 96, 256, generator=g).bfloat16() * (1 + i) for i in range(5)]
    for gran in ('per_tensor', 'per_token'):
        spec = Q.IntSpec(8, True, gran)
        q = IntegerQuantizer(8, True, gran, calib_algo='static_minmax')
        lo, hi = q.get_static_minmax_range([a.to(dev) for a in acts])
        olo, ohi = Q.static_minmax_ranges(spec, list(acts))
        assert_bit_equal(lo[0], olo[0], 'static min'); assert_bit_equal(hi[0], ohi[0], 'static max')
        sl, zl, qminl, qmaxl = q.get_batch_tensors_qparams([a.to(dev) for a in acts])
        os_, oz, oqmax, oqmin = Q.int_qparams(spec, olo[0], ohi[0])
        assert len(sl) == 1 and and_bit(sl[0], os_) and float(qmaxl[0]) == float(oqmax) and float(qminl[0]) == float(oqmin)
        q = IntegerQuantizer(8, True, gran, calib_algo='static_moving_minmax')
        lo, hi = q.get_static_moving_minmax_range([a.to(dev) for a in acts], 0.3)
        olo, ohi = Q.static_moving_minmax_ranges(spec, list(acts), 0.3)
        assert_bit_equal(lo[0], olo[0], 'moving min'); assert_bit_equal(hi[0], ohi[0], 'moving max')
        sl, _, _, _ = q.get_batch_tensors_qparams([a.to(dev) for a in acts], alpha=0.3)
        assert and_bit(sl[0], Q.int_qparams(spec, olo[0], ohi[0])[0])
    # asymmetric, tuple inputs (two module inputs), batch-in-one-tensor
    spec = Q.IntSpec(8, False, 'per_tensor')
    q = IntegerQuantizer(8, False, 'per_tensor', calib_algo='static_minmax')
    pairs = [(acts[0][0], acts[1][0]), (acts[2][0], acts[3][0])]
    sl, zl, _, _ = q.get_batch_tensors_qparams([(a.to(dev), b.to(dev)) for a, b in pairs])
    olo, ohi = Q.static_minmax_ranges(spec, pairs)
    assert len(sl) == 2
    for i in range(2):
        os_, oz, _, _ = Q.int_qparams(spec, olo[i], ohi[i])
        assert and_bit(sl[i], os_) and and_bit(zl[i], oz)
    lo, hi = q.get_static_minmax_range([acts[0].to(dev)])
    olo, ohi = Q.static_minmax_ranges(spec, [acts[0]])
    assert_bit_equal(lo[0], olo[0], 'batch tensor min')
    with pytest.raises(AssertionError):                       # quant.py:563-566: per-tensor symmetric only
        IntegerQuantizer(8, False, 'per_tensor', calib_algo='static_hist').get_batch_tensors_qparams([acts[0].to(dev)])


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_histogram_kernel(dev, dtype):
    """lcq_histc against the device binning formula of torch.histc: counts identical, for ragged lengths, values on
    and outside the edges, a constant tensor (range widened by one), and more than 2^24 hits in one bin."""
    from lightcompress_amd import IntegerQuantizer
    q = IntegerQuantizer(8, True, 'per_tensor', calib_algo='static_hist')
    g = gen(21)
    for n, bins in [(100003, 2048), (4096 * 33 + 5, 512), (7, 16)]:
        q.bins = bins
        x = (torch.randn(n, generator=g) * 3).to(dtype)
        lo, hi = float(x.min()), float(x.max())
        for a, b in [(lo, hi), (lo * 0.5, hi * 0.25), (lo - 1.0, hi + 2.5)]:
            got = q._histc(x.to(dev), a, b)
            want = Q.histc_device(x, bins, a, b)
            assert torch.equal(got, want), (n, bins, a, b, int((got != want).sum()))
            # torch's own GPU kernel, as the reference calls it (quant.py:473-487): pins the binning formula itself
            on_gpu = torch.histc(x.to(dev).float(), bins=bins, min=a, max=b).cpu()
            assert torch.equal(got, on_gpu), (n, bins, a, b, int((got != on_gpu).sum()))
    if dtype == torch.float32:
        # Values on and one ulp to either side of every bin edge of a range that is no power of two: here the order of
        # the multiply and the divide matters (hundreds of these values change bin with the divide first), so equality
        # with torch.histc on the GPU pins the order.
        import numpy as np
        a, b = 0.3, 7.1
        for bins in (1000, 333):
            e = (a + np.arange(bins + 1, dtype=np.float64) * (b - a) / bins).astype(np.float32)
            v = np.concatenate([e, np.nextafter(e, np.float32(100)), np.nextafter(e, np.float32(-100))])
            a32, b32 = np.float32(a), np.float32(b)
            vi = v[(v >= a32) & (v <= b32)]
            differ = (((vi - a32) * np.float32(bins) / (b32 - a32)).astype(np.int64)
                      != ((vi - a32) / (b32 - a32) * np.float32(bins)).astype(np.int64)).sum()
            assert differ >= 50, differ
            q.bins = bins
            xe = torch.from_numpy(v)
            got = q._histc(xe.to(dev), a, b)
            assert torch.equal(got, torch.histc(xe.to(dev), bins=bins, min=a, max=b).cpu()), bins
            assert torch.equal(got, Q.histc_device(xe, bins, a, b)), bins
    q.bins = 64
    c = torch.full((1000,), 2.5, dtype=dtype)
    assert torch.equal(q._histc(c.to(dev), 2.5, 2.5), Q.histc_device(c, 64, 2.5, 2.5))
    assert torch.equal(q._histc(c.to(dev), 2.5, 2.5), torch.histc(c.to(dev).float(), bins=64, min=2.5, max=2.5).cpu())
    if dtype == torch.bfloat16:
        big = torch.zeros(1 << 25, dtype=dtype, device=dev)
        big[::1024] = 1.0
        h = q._histc(big, 0.0, 1.0)
        assert float(h[0]) == float((1 << 25) - (1 << 15)) and float(h[63]) == float(1 << 15) and float(h[1:63].sum()) == 0.0


def test_static_hist_calibration(dev):
    """calib_algo='static_hist' (quant.py:264-521, 563-567): the thresholded range and the qparams equal the oracle's
    bit for bit - tensors of growing range (the histogram is re-binned), of equal range, a batch in one tensor, two
    module inputs, fp32 and bf16 activations."""
    from lightcompress_amd import IntegerQuantizer
    g = gen(31)
    spec = Q.IntSpec(8, True, 'per_tensor')
    grow = [torch.randn(2, 200, 128, generator=g).bfloat16() * (1 + i) for i in range(4)]
    same = [torch.randn(300, 64, generator=g).clamp(-2, 2) for _ in range(3)]
    for t in same:
        t[0, 0], t[0, 1] = -2.0, 2.0
    shrink = [torch.randn(128, 96, generator=g) * s for s in (4.0, 1.0, 2.0)]
    for acts in (grow, same, shrink, [grow[0]]):
        q = IntegerQuantizer(8, True, 'per_tensor', calib_algo='static_hist')
        lo, hi = q.get_static_hist_range([a.to(dev) for a in acts])
        olo, ohi = Q.static_hist_ranges([a.clone() for a in acts], 8)
        assert len(lo) == len(olo) == 1
        assert_bit_equal(lo[0], olo[0], 'hist min'); assert_bit_equal(hi[0], ohi[0], 'hist max')
        sl, zl, qminl, qmaxl = q.get_batch_tensors_qparams([a.to(dev) for a in acts])
        os_, oz, oqmax, oqmin = Q.int_qparams(spec, olo[0], ohi[0])
        assert and_bit(sl[0], os_) and float(qmaxl[0]) == 127.0 and float(qminl[0]) == -128.0
    pairs = [(grow[0][0], same[0]), (grow[1][0], same[1])]
    q = IntegerQuantizer(4, True, 'per_tensor', calib_algo='static_hist', bins=512)
    sl, _, _, _ = q.get_batch_tensors_qparams([(a.to(dev), b.to(dev)) for a, b in pairs])
    olo, ohi = Q.static_hist_ranges(pairs, 4, bins=512)
    spec4 = Q.IntSpec(4, True, 'per_tensor')
    assert len(sl) == 2 and and_bit(sl[0], Q.int_qparams(spec4, olo[0], ohi[0])[0]) and and_bit(sl[1], Q.int_qparams(spec4, olo[1], ohi[1])[0])


def and_bit(a, b):
    assert_bit_equal(a.cpu(), b, 'qparam')
    return True


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('b4,b8,shape', [
    (dict(symmetric=False, granularity='per_group', group_size=128), dict(symmetric=True, granularity='per_channel'), (64, 1024)),
    (dict(symmetric=True, granularity='per_group', group_size=64, scales_bit=8, scales_symmetric=False),
     dict(symmetric=False, granularity='per_channel'), (48, 512)),
    (dict(symmetric=False, granularity='per_group', group_size=32, scales_bit=2, scales_symmetric=False),
     dict(symmetric=True, granularity='per_group', group_size=256), (32, 512)),
])
def test_weight48_fake_quant_bit_exact(dev, dtype, b4, b8, shape):
    """Weight48IntegerQuantizer.fake_quant_weight_dynamic (quant.py:1338-1367) against its oracle, bit for bit."""
    from lightcompress_amd.quant import Weight48IntegerQuantizer
    w = weight_like(*shape, seed=shape[1], dtype=dtype)
    q = Weight48IntegerQuantizer(48, dict(b4), dict(b8))
    got = q.fake_quant_weight_dynamic(w.to(dev))
    want = Q.w48_fake_quant(w, b4, b8)
    assert_bit_equal(got, want, 'w48 fake quant')


@pytest.mark.parametrize('m', [1, 2, 4, 8])
def test_stream_probe_reads_everything_and_refuses_a_short_destination(dev, m):
    """The benchmark's streaming probe: every 16-byte chunk of the source reaches the output (xor of m chunks of a
    thread's share), and a destination smaller than bytes / m is refused on the host."""
    from lightcompress_amd import _lib as L
    u = 4 if m < 4 else m                                   # chunks per thread
    nblocks = 37
    g = torch.Generator().manual_seed(m)
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (nblocks, u // m, m, 256, 4), generator=g, dtype=torch.int64).to(torch.int32)
    want = src[:, :, 0]
    for k in range(1, m):
        want = want ^ src[:, :, k]
    sd = src.to(dev).contiguous()
    out = torch.zeros(want.numel(), dtype=torch.int32, device=dev)
    nbytes = sd.numel() * 4
    L.check(L.lib().lcq_stream_probe(L.ptr(sd), L.ptr(out), L.i64(nbytes), L.i64(out.numel() * 4), L.i32(m), L.stream()), 'probe')
    assert torch.equal(out.cpu(), want.reshape(-1))
    with pytest.raises(L.LcqError):
        L.check(L.lib().lcq_stream_probe(L.ptr(sd), L.ptr(out), L.i64(nbytes), L.i64(out.numel() * 4 - 16), L.i32(m), L.stream()),
                'probe')
    with pytest.raises(L.LcqError):
        L.check(L.lib().lcq_stream_probe(L.ptr(sd), L.ptr(out), L.i64(nbytes), L.i64(out.numel() * 4), L.i32(3), L.stream()), 'probe')
    # read-only pass: nothing is written
    out.zero_()
    L.check(L.lib().lcq_stream_probe(L.ptr(sd), L.ptr(out), L.i64(nbytes), L.i64(out.numel() * 4), L.i32(0), L.stream()), 'probe')
    assert int(out.abs().sum()) == 0


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_int_static_activation_fake_quant_plain_and_mixed_precision(dev, dtype):
    """fake_quant_act_static (quant.py:718-751) with parameters calibrated beforehand: the whole tensor, and the
    mixed-precision form in which `int_indices` columns are quantized and `fp_indices` columns pass through."""
    act = (torch.randn(3, 40, 256, generator=gen(901)) * 2).to(dtype)
    spec = Q.IntSpec(8, True, 'per_tensor')
    q = _iq(8, True, 'per_tensor')
    calib = (torch.randn(3, 40, 256, generator=gen(902)) * 2).to(dtype)
    _, s, z, qmax, qmin = Q.int_tensor_qparams(spec, calib)
    args = dict(scales=s.to(dev), zeros=z.to(dev) if torch.is_tensor(z) else z, qmax=qmax, qmin=qmin, current_bit=4)
    got = q.fake_quant_act_static(act.to(dev), dict(args))
    want = Q.int_fake_quant_static(spec, act, s, z, qmax, qmin)
    assert_bit_equal(got, want, 'fake_quant_act_static')
    assert q.bit == 8
    perm = torch.randperm(256, generator=gen(903))
    ii, fi = perm[:192].sort().values, perm[192:].sort().values
    mixed = q.fake_quant_act_static(act.to(dev), dict(args, int_indices=ii.to(dev), fp_indices=fi.to(dev)))
    want_q = Q.int_fake_quant_static(spec, act[:, :, ii].contiguous(), s, z, qmax, qmin)
    assert_bit_equal(mixed[:, :, ii.to(dev)], want_q, 'quantized columns')
    assert_bit_equal(mixed[:, :, fi.to(dev)], act[:, :, fi], 'columns kept in floating point')


def test_mixed_precision_indices_in_the_dynamic_paths(dev):
    """`int_indices` / `fp_indices` (quant.py:753-782 activations, :832-868 weights): the named columns are quantized
    as a tensor of their own, the others pass through."""
    act = (torch.randn(2, 24, 384, generator=gen(911)) * 2).bfloat16()
    perm = torch.randperm(384, generator=gen(912))
    ii, fi = perm[:256].sort().values, perm[256:].sort().values
    aq = _iq(8, True, 'per_token')
    mixed = aq.fake_quant_act_dynamic(act.to(dev), dict(int_indices=ii.to(dev), fp_indices=fi.to(dev)))
    want = Q.int_fake_quant_dynamic(Q.IntSpec(8, True, 'per_token'), act[:, :, ii].contiguous())
    assert_bit_equal(mixed[:, :, ii.to(dev)], want, 'quantized activation columns')
    assert_bit_equal(mixed[:, :, fi.to(dev)], act[:, :, fi], 'activation columns kept')
    w = weight_like(64, 384, seed=913, dtype=torch.bfloat16)
    wq = _iq(4, False, 'per_group', group_size=128)
    mixed = wq.fake_quant_weight_dynamic(w.to(dev), dict(int_indices=ii.to(dev), fp_indices=fi.to(dev)))
    want = Q.int_fake_quant_dynamic(Q.IntSpec(4, False, 'per_group', group_size=128), w[:, ii].contiguous())
    assert_bit_equal(mixed[:, ii.to(dev)], want, 'quantized weight columns')
    assert_bit_equal(mixed[:, fi.to(dev)], w[:, fi], 'weight columns kept')


def test_experts_in_one_launch_equal_expert_by_expert(dev):
    """Several experts through one launch (their rows stacked): float8 real quant, int4 real quant and int4 quantize +
    pack give every expert what its own call gives, bit for bit; consecutive slices of one tensor are stacked as a view."""
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer
    from lightcompress_amd.quant import experts_as_rows
    E, R, K = 5, 96, 1024
    stacked = weight_like(E * R, K, seed=77, dtype=torch.bfloat16, std=0.006, outlier_frac=0.001, outlier_mul=30).to(dev).view(E, R, K)
    slices = [stacked[e] for e in range(E)]
    apart = [s.clone() for s in slices]
    assert experts_as_rows(slices).data_ptr() == stacked.data_ptr()           # a view
    assert experts_as_rows(apart).data_ptr() not in [a.data_ptr() for a in apart]
    assert torch.equal(experts_as_rows(apart), stacked.view(E * R, K))
    fq = FloatQuantizer('e4m3', True, 'per_channel', use_qtorch=True)
    iq = IntegerQuantizer(4, True, 'per_group', group_size=128)
    ia = IntegerQuantizer(4, False, 'per_group', group_size=128)
    for ws in (slices, apart):
        for q in (fq, iq, ia):
            many = q.real_quant_weight_dynamic_experts(ws)
            for e in range(E):
                one = q.real_quant_weight_dynamic(ws[e])
                for a, b in zip(many[e], one):
                    assert (a is None and b is None) or (a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a,
                                                                                       b.view(torch.uint8) if b.dtype == torch.float8_e4m3fn else b))
        many = iq.real_quant_pack_dynamic_experts(ws)
        for e in range(E):
            one = iq.real_quant_pack_dynamic(ws[e])
            assert torch.equal(many[e][0], one[0]) and torch.equal(many[e][1], one[1])
    with pytest.raises(NotImplementedError):
        IntegerQuantizer(4, True, 'per_tensor').real_quant_weight_dynamic_experts(slices)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('shape', [(256, 384), (200, 300)])
def test_float_per_block_with_given_scales(dev, dtype, shape):
    """FloatQuantizer('e4m3', per_block) with static scales (the block scales of a float8 checkpoint, or those of an
    earlier dynamic call): fake and real quantization bit for bit against the oracle, ragged shapes padded with zeros
    like reshape_tensor does, a zero scale replaced by 1 in the caller's tensor; with the scales of its own dynamic
    call the static path reproduces the dynamic one."""
    from lightcompress_amd import FloatQuantizer
    m, n = shape
    w = weight_like(m, n, seed=m + n, dtype=dtype, std=0.02, outlier_frac=0.002, outlier_mul=20)
    mb, nb = -(-m // 128), -(-n // 128)
    scales = (torch.rand(mb, 1, nb, 1, generator=gen(5)) * 4e-4 + 1e-4)
    scales[0, 0, 0, 0] = 0.0
    spec = Q.FloatSpec('e4m3', 'per_block')
    q = FloatQuantizer('e4m3', True, 'per_block', use_qtorch=True, block_size=128)
    sd = scales.clone().to(dev)
    got = q.fake_quant_weight_static(w.to(dev), {'scales': sd, 'zeros': torch.tensor(0.0), 'qmax': q.qmax, 'qmin': q.qmin})
    so = scales.clone()
    assert_bit_equal(got, Q.float_per_block_static(spec, w, so), 'static per_block fake quant')
    assert float(sd[0, 0, 0, 0]) == 1.0 and float(so[0, 0, 0, 0]) == 1.0          # both mutated the caller's scales
    codes, rs, rz = q.real_quant_weight_static(w.to(dev), {'scales': sd, 'zeros': torch.tensor(0.0), 'qmax': q.qmax, 'qmin': q.qmin})
    assert rz is None and rs.shape == (mb, nb) and codes.dtype == torch.float8_e4m3fn and codes.shape == (m, n)
    assert_bit_equal(codes, Q.float_per_block_static(spec, w, so, real=True), 'static per_block codes')
    # the scales of the dynamic call, handed back: the same codes (ragged widths go through a zero-padded copy)
    dyn_codes, dyn_s, _ = q.real_quant_weight_dynamic(w.to(dev))
    again, _, _ = q.real_quant_weight_static(w.to(dev), {'scales': dyn_s.view(mb, 1, nb, 1).clone(), 'zeros': torch.tensor(0.0),
                                                         'qmax': q.qmax, 'qmin': q.qmin})
    assert_bit_equal(again, dyn_codes, 'static with the dynamic scales')
    oc, os_, _ = Q.float_per_block_real_quant(spec, w)
    assert_bit_equal(dyn_codes, oc, 'dynamic per_block codes'); assert_bit_equal(dyn_s, os_, 'dynamic per_block scales')
    assert_bit_equal(q.fake_quant_weight_dynamic(w.to(dev)), Q.float_per_block_static(spec, w, os_.view(mb, 1, nb, 1).clone()), 'dynamic per_block fake quant')


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('sym', [True, False])
def test_int_infinite_and_nan_weights_propagate_like_torch(dev, dtype, sym):
    """An infinite weight makes its group's scale infinite: every dequantized value of the group is 0 * inf = NaN, the
    infinite element's own code is round(inf / inf) = NaN, which torch.clamp hands on; a NaN weight turns the range
    and with it the whole group into NaN.  Groups without such a weight are untouched."""
    for bad in (float('inf'), float('-inf'), float('nan')):
        w = weight_like(16, 512, seed=77, dtype=dtype)
        w[3, 130] = bad
        spec = Q.IntSpec(4, sym, 'per_group', group_size=128)
        got = _iq(4, sym, 'per_group', group_size=128).fake_quant_weight_dynamic(w.to(dev)).cpu()
        want = Q.int_fake_quant_dynamic(spec, w)
        assert torch.equal(torch.isnan(got), torch.isnan(want)), bad
        assert torch.equal(torch.nan_to_num(got.float(), 0.0, 1e30, -1e30), torch.nan_to_num(want.float(), 0.0, 1e30, -1e30)), bad
        assert bool(torch.isnan(want[3, 128:256]).all()) or not sym


def test_fp16_output_scale_factor_rounds_twice_like_torch(dev):
    """scales * output_scale_factor on fp16 scales: torch forms the fp32 product, rounds it, then converts to fp16.
    A multiply fused with the conversion rounds the exact product once, and the two disagree when the fp32 rounding lands
    on an fp16 tie: s = 845 * 2^-11 times 1.7 is 1436.5 * 2^-11 after the fp32 rounding (1.7 is 1.70000005 in fp32, the
    exact product lies just above the tie).  Scales built to sit on such ties, for the dequantized values and for the
    scales real_quant_weight_static returns."""
    k = torch.arange(5, 2048, 10)                                         # k * 1.7 = n + 0.5
    s = (k.float() * 2.0 ** -11).to(torch.float16).reshape(-1, 1)
    # k = 845: the exact product lies above the tie 1436.5 * 2^-11, torch's two roundings end on the even neighbour below
    assert 845 * 2.0 ** -11 * 1.7000000476837158 > 1436.5 * 2.0 ** -11
    assert float((s * 1.7)[84]) == 1436 * 2.0 ** -11 and float(s[84]) == 845 * 2.0 ** -11
    R = s.shape[0]
    x = (torch.randn(R, 64, generator=gen(5)) * 3).to(torch.float16)
    z = torch.full((R, 1), 8.0, dtype=torch.float16)
    spec = Q.IntSpec(4, False, 'per_channel')
    q = _iq(4, False, 'per_channel')
    args = dict(scales=s.to(dev), zeros=z.to(dev), qmax=spec.qmax, qmin=spec.qmin, output_scale_factor=1.7)
    assert_bit_equal(q.fake_quant_weight_static(x.to(dev), dict(args)),
                     Q.int_fake_quant_static(spec, x, s, z, spec.qmax, spec.qmin, output_scale_factor=1.7), 'dequantized values')
    codes, rs, rz = q.real_quant_weight_static(x.to(dev), dict(args))
    ocodes, ors, orz = Q.int_real_quant_static(spec, x, s, z, spec.qmax, spec.qmin, output_scale_factor=1.7)
    assert_bit_equal(codes, ocodes, 'codes')
    assert_bit_equal(rs, ors, 'returned scales')
