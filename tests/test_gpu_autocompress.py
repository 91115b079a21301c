"""GPU parity: single-layer fused Linear, FusedCompressor, the bias-free generated MLP, sparse gather and the
per-row quantiser (the kernel factories of the reference) vs the CPU oracle.

Tolerances: gathers and quantiser codes/scales/de-quantised values are bit-exact.  GEMM results follow the bar of
the CCM MLP tests (error norm <= 1e-3 of the reference norm, every element within 1e-3 * max|ref| + 2 ulp of the
storage dtype): both sides accumulate in fp32 and round once per Linear, in a different summation order.
"""
import pytest
import torch

from fastcache_amd import autocompress as ac
from fastcache_amd import ops
from fastcache_amd._lib import FastcacheError
from fastcache_amd.kernels import FusedCompressor, fused_linear_relu_dropout
from oracle import autocompress as oa
from oracle import ccm as occm

from test_gpu_ccm import assert_mlp_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,N,bias,relu", [(1000, 640, 128, True, True), (33, 256, 96, True, False),
                                             (5, 16, 32, False, True), (257, 128, 160, True, True),
                                             (4096, 256, 128, True, True)])
def test_linear_act(dev, dtype, M, K, N, bias, relu):
    g = torch.Generator().manual_seed(M + K + N)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(K, N, generator=g) / K ** 0.5).to(dtype)
    b = torch.randn(N, generator=g).to(dtype) if bias else None
    ref = oa.linear_act(x, w, b, relu)
    got = ops.linear_act(x.to(dev), w.t().contiguous().to(dev), None if b is None else b.to(dev), relu)
    assert got.shape == (M, N) and got.dtype == dtype
    assert_mlp_close(got.cpu(), ref, dtype)
    # the reference's call signature: weight [K, N]
    got2 = fused_linear_relu_dropout(x.to(dev), w.to(dev), (b if b is not None else torch.zeros(N, dtype=dtype)).to(dev),
                                     dropout_p=0.4, apply_relu=relu, training=False)
    assert torch.equal(got2, got)


def test_linear_act_rejects_what_it_cannot_do(dev):
    x = torch.randn(8, 24, dtype=torch.float16, device=dev)
    with pytest.raises(FastcacheError):
        ops.linear_act(x, torch.randn(32, 24, dtype=torch.float16, device=dev), None, True)      # K % 16
    with pytest.raises(FastcacheError):
        ops.linear_act(x.float(), torch.randn(32, 24, device=dev), None, True)                   # fp32
    with pytest.raises(FastcacheError):
        fused_linear_relu_dropout(torch.randn(8, 32, dtype=torch.float16, device=dev),
                                  torch.randn(32, 32, dtype=torch.float16, device=dev),
                                  torch.zeros(32, dtype=torch.float16, device=dev), dropout_p=0.4, training=True)


@pytest.mark.parametrize("dtype,cf,S", [(torch.float16, 5, 603), (torch.bfloat16, 2, 64), (torch.float16, 5, 3)])
def test_fused_compressor_layer(dev, dtype, cf, S):
    from fastcache_amd.utils_ccm import KVCacheHybridCompressor
    from types import SimpleNamespace
    L, B, H, D = 3, 2, 4, 128
    cfg = SimpleNamespace(architectures=["MiniCPMV"], num_hidden_layers=L, num_key_value_heads=H,
                          num_attention_heads=H, hidden_size=H * D)
    torch.manual_seed(3)
    module = KVCacheHybridCompressor(cfg, compression_factor=cf, min_seq_len=1).to(dev).to(dtype).eval()
    fc = FusedCompressor(num_layers=L, num_heads=H, head_dim=D, compression_factor=cf)
    fc.load_from_pytorch_module(module)
    assert fc.w1_k.shape == (L, cf * D, D) and fc.w1_k.device.type == "cuda"
    g = torch.Generator().manual_seed(11)
    k = torch.randn(B, H, S, D, generator=g).to(dtype)
    v = torch.randn(B, H, S, D, generator=g).to(dtype)
    layer = 1
    gk, gv = fc.compress_layer_fused(k.to(dev), v.to(dev), layer)
    for got, src, grp in ((gk, k, "k"), (gv, v, "v")):
        w = tuple(getattr(fc, f"{n}{i}_{grp}")[layer].cpu() for i in (1, 2, 3) for n in ("w", "b"))
        ref = oa.fused_compress_layer(src, w, cf)
        assert got.shape == ref.shape
        c = S // cf
        if c >= 1:
            assert_mlp_close(got[:, :, :c].cpu(), ref[:, :, :c], dtype)
            assert torch.equal(got[:, :, c:].cpu(), ref[:, :, c:])          # remainder tokens copied through
        else:
            assert torch.equal(got.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,N", [(700, 640, 128), (129, 256, 128), (50, 64, 64)])
def test_generated_mlp_kernel(dev, dtype, M, K, N):
    g = torch.Generator().manual_seed(M)
    X = torch.randn(M, K, generator=g).to(dtype)
    W1 = (torch.randn(K, N, generator=g) / K ** 0.5).to(dtype)
    W2 = (torch.randn(N, N, generator=g) / N ** 0.5).to(dtype)
    W3 = (torch.randn(N, N, generator=g) / N ** 0.5).to(dtype)
    fn = ac.get_mlp_kernel(M, N, K, "float16" if dtype == torch.float16 else "bfloat16")
    got = fn(X.to(dev), W1.to(dev), W2.to(dev), W3.to(dev))
    assert_mlp_close(got.cpu(), oa.mlp_nobias(X, W1, W2, W3), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_sparse_gather_bit_exact(dev, dtype):
    g = torch.Generator().manual_seed(2)
    X = torch.randn(777, 128, generator=g).to(dtype)
    idx = torch.sort(torch.randperm(777, generator=g)[:200]).values
    fn = ac.get_sparse_gather_kernel()
    got = fn(X.to(dev), idx.to(dev))
    assert torch.equal(got.cpu(), oa.sparse_gather(X, idx))
    assert fn(X.to(dev), idx[:0].to(dev)).shape == (0, 128)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(3, 5, 128), (7, 40), (1000, 128)])
def test_quantize_dequantize_bit_exact(dev, dtype, bits, shape):
    g = torch.Generator().manual_seed(bits + len(shape))
    X = (torch.randn(*shape, generator=g) * 2.5).to(dtype)
    X.view(-1, shape[-1])[0, 3] = 40.0            # an outlier row
    quant, dequant = ac.get_quantize_kernels(bits)
    q, sc = quant(X.to(dev))
    rq, rsc = oa.quantize(X, bits)
    assert q.dtype == torch.int8 and sc.dtype == dtype and sc.shape == rsc.shape
    assert torch.equal(sc.cpu(), rsc)
    assert torch.equal(q.cpu(), rq)
    for out_dtype in (dtype, torch.float32):
        got = dequant(q, sc, out_dtype)
        ref = oa.dequantize(rq, rsc, out_dtype)
        assert got.dtype == ref.dtype and torch.equal(got.cpu(), ref)


def test_hardware_profile_and_streams(dev):
    prof = ac.detect_hardware()
    assert prof.gpu_arch == ac.GPUArch.CDNA4 and prof.memory_bandwidth_gbps == 8000.0
    assert abs(ac.get_hardware_profile("MI355X").roofline_intensity - 312.5) < 1e-9
    with pytest.raises(ValueError):
        ac.get_hardware_profile("no-such-gpu")
    sm = ac.get_stream_manager()
    side = sm.get_compress_stream()
    assert side is not None and side != sm.get_main_stream() and side.priority == 0
    x = torch.zeros(1 << 20, device=dev)
    with torch.cuda.stream(side):
        x += 1
    sm.synchronize_compress_to_main()
    assert float((x * 2).sum()) == 2.0 * (1 << 20)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["int8", "int4", "nf4"])
def test_quantization_method_bit_exact(dev, dtype, kind):
    """QuantizationMethod (int8 per row, int4 / NF4 per group of 128, two codes per byte) against the oracle:
    codes, scales and de-quantised values bit for bit."""
    g = torch.Generator().manual_seed(len(kind))
    X = (torch.randn(2, 3, 50, 128, generator=g) * 1.7).to(dtype)
    V = (torch.randn(2, 3, 50, 128, generator=g) * 0.3).to(dtype)
    qm = ac.QuantizationMethod(kind, group_size=128)
    (qk, sk), (qv, sv) = qm.compress(X.to(dev), V.to(dev))
    for x, q, s in ((X, qk, sk), (V, qv, sv)):
        if kind == "int8":
            rq, rs = oa.quantize_int8(x)
            ref = oa.dequantize(rq, rs, dtype)
        else:
            rq, rs = (oa.quantize_int4 if kind == "int4" else oa.quantize_nf4)(x, 128)
            ref = oa.dequantize_4bit(rq, rs, 128, kind == "nf4", dtype)
        assert q.dtype == rq.dtype and q.shape == rq.shape and torch.equal(q.cpu(), rq)
        assert s.dtype == dtype and s.shape == rs.shape and torch.equal(s.cpu(), rs)
        got = qm.dequantize(q, s, dtype)
        assert got.dtype == ref.dtype and torch.equal(got.cpu(), ref)
    assert qm.name == f"quant_{kind}" and qm.compression_ratio == (2.0 if kind == "int8" else 4.0)
    # several groups per row
    if kind != "int8":
        qm2 = ac.QuantizationMethod(kind, group_size=32)
        q, s = qm2._quantize(X.to(dev))
        rq, rs = (oa.quantize_int4 if kind == "int4" else oa.quantize_nf4)(X, 32)
        assert s.shape == (2, 3, 50, 4) and torch.equal(q.cpu(), rq) and torch.equal(s.cpu(), rs)
        assert torch.equal(qm2.dequantize(q, s, dtype).cpu(), oa.dequantize_4bit(rq, rs, 32, kind == "nf4", dtype))


def _fp8_bits(t):
    return t.view(torch.uint8)


@pytest.mark.parametrize("e5m2", [False, True])
def test_fp8_cast_every_half_and_bfloat_value(dev, e5m2):
    """Every fp16 and every bf16 bit pattern with |x| <= 448, in a tensor whose largest magnitude is 448 so that the
    scale is exactly 1: the codes are the float8 cast itself, compared with torch's CPU cast bit for bit
    (subnormal targets, ties, both signs, zeros)."""
    for dtype in (torch.float16, torch.bfloat16):
        allv = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        x = allv[allv.float().abs() <= 448]
        assert float(x.float().abs().max()) == 448.0 and x.numel() > 30000
        q, s = ops.quantize_fp8(x.to(dev), e5m2=e5m2)
        rq, rs = oa.quantize_fp8(x, e5m2)
        assert float(s) == 1.0 and float(rs.reshape(-1)[0]) == 1.0
        assert q.dtype == rq.dtype and torch.equal(_fp8_bits(q.cpu()), _fp8_bits(rq))
        # and back: every code times a scale
        sc = torch.tensor(0.37, dtype=dtype)
        got = ops.dequantize_fp8(q, sc.to(dev), dtype)
        assert torch.equal(got.cpu(), oa.dequantize_fp8(rq, sc, dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["fp8", "fp8_e4m3", "fp8_e5m2"])
def test_quantization_method_fp8_bit_exact(dev, dtype, kind):
    """QuantizationMethod fp8: float8 codes, the expanded whole-tensor scale and the de-quantised values against
    the eager expressions on the CPU, bit for bit; fp32 inputs reach the cast unrounded."""
    g = torch.Generator().manual_seed(len(kind) + 3)
    X = (torch.randn(2, 3, 50, 128, generator=g) * 1.7).to(dtype)
    V = (torch.randn(2, 3, 50, 128, generator=g) * torch.logspace(-6, 1, 128)).to(dtype)   # reaches float8 subnormals
    qm = ac.QuantizationMethod(kind)
    e5m2 = kind == "fp8_e5m2"
    (qk, sk), (qv, sv) = qm.compress(X.to(dev), V.to(dev))
    for x, q, s in ((X, qk, sk), (V, qv, sv)):
        rq, rs = oa.quantize_fp8(x, e5m2)
        assert q.dtype == rq.dtype and q.shape == rq.shape and torch.equal(_fp8_bits(q.cpu()), _fp8_bits(rq))
        assert s.dtype == dtype and s.shape == rs.shape == x.shape[:-1] + (1,) and torch.equal(s.cpu(), rs)
        for out_dtype in (dtype, torch.float32):
            got = qm.dequantize(q, s, out_dtype)
            ref = oa.dequantize_fp8(rq, rs, out_dtype)
            assert got.dtype == ref.dtype and torch.equal(got.cpu(), ref)
    assert qm.name == ("quant_fp8_e5m2" if e5m2 else "quant_fp8_e4m3") and qm.compression_ratio == 2.0


def test_fp8_special_tensors(dev):
    """An all-zero tensor (scale floored at 1e-8, or at 0 in fp16 where 1e-8 underflows: 0/0 = NaN codes), a NaN in
    the tensor (every code NaN), one element."""
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for x in (torch.zeros(4, 8), torch.tensor([[1.0, float("nan"), -2.0, 0.5]]), torch.tensor([[-3.0]])):
            x = x.to(dtype)
            q, s = ops.quantize_fp8(x.to(dev))
            rq, rs = oa.quantize_fp8(x)
            assert torch.equal(q.cpu().float().isnan(), rq.float().isnan())
            ok = ~rq.float().isnan()
            assert torch.equal(_fp8_bits(q.cpu())[ok], _fp8_bits(rq)[ok])
            assert torch.equal(s.cpu().reshape(-1)[:1].float().nan_to_num(-1.0), rs.reshape(-1)[:1].float().nan_to_num(-1.0))
    with pytest.raises(FastcacheError):
        ops.dequantize_fp8(torch.zeros(4, dtype=torch.int8, device=dev), torch.ones((), device=dev), torch.float16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 5, 128), (7, 40), (1000, 128), (2, 1)])
def test_quantization_method_asymmetric_int8_bit_exact(dev, dtype, shape):
    """symmetric=False: uint8 codes, scale and zero point per row against the eager expression; rows that are
    constant (scale floored), all positive, all negative."""
    g = torch.Generator().manual_seed(shape[0])
    x = (torch.randn(*shape, generator=g) * 2.5 + 0.7).to(dtype)
    x[0] = 1.25
    if shape[0] > 2:
        x[1] = x[1].abs() + 0.5
        x[2] = -x[2].abs() - 0.5
    qm = ac.QuantizationMethod("int8", symmetric=False)
    q, p = qm._quantize(x.to(dev))
    rq, rp = oa.quantize_int8_asymmetric(x)
    assert q.dtype == torch.uint8 and q.shape == rq.shape and torch.equal(q.cpu(), rq)
    assert p.dtype == dtype and p.shape == rp.shape == x.shape[:-1] + (2,)
    assert torch.equal(p.cpu()[..., 0], rp[..., 0])
    assert bool((p.cpu()[..., 1].float() == rp[..., 1].float()).all())        # +0 and -0 compare equal
    with pytest.raises(FastcacheError):
        qm.dequantize(q, p, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("per_tensor", [False, True])
def test_fake_quantize_bit_exact(dev, dtype, bits, per_tensor):
    """fc_fake_quantize against the eager expression of SimpleKVQuantizer / ImprovedKVQuantizer, bit for bit."""
    from oracle import presses as op
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(2, 4, 300, 128, generator=g) * 2.5).to(dtype)
    x[0, 1, 7] = 0                                       # an all-zero row: NaN per row, plain zeros per tensor
    ref, rsc, rmx = op.fake_quantize(x, bits, per_tensor)
    got, sc, mx = ops.fake_quantize(x.to(dev), bits, per_tensor, return_params=True)
    assert torch.equal(torch.nan_to_num(sc.cpu().view(rsc.shape).float(), nan=-1), torch.nan_to_num(rsc.float(), nan=-1))
    assert torch.equal(torch.nan_to_num(mx.cpu().view(rmx.shape).float(), nan=-1), torch.nan_to_num(rmx.float(), nan=-1))
    assert torch.equal(torch.isnan(got.cpu()), torch.isnan(ref))
    assert torch.equal(torch.nan_to_num(got.cpu().float(), nan=0.0), torch.nan_to_num(ref.float(), nan=0.0))
    # in place
    xd = x.to(dev).clone()
    ops.fake_quantize(xd, bits, per_tensor, out=xd)
    assert torch.equal(torch.nan_to_num(xd.cpu().float(), nan=0.0), torch.nan_to_num(ref.float(), nan=0.0))


def test_fake_quantize_large_tensor_and_nan(dev):
    """More elements than one pass of the partial maxima covers; a NaN anywhere poisons the whole-tensor scale."""
    from oracle import presses as op
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 1024, 1024, generator=g).half()
    x[2, 1000, 1000] = 40.0                               # the maximum sits near the end
    ref = op.fake_quantize(x, 4, True)[0]
    got = ops.fake_quantize(x.to(dev), 4, True).cpu()
    assert torch.equal(got, ref)
    x[1, 5, 5] = float("nan")
    assert torch.isnan(ops.fake_quantize(x.to(dev), 4, True)).all()


def test_kv_quantizer_objects(dev):
    """SimpleKVQuantizer / ImprovedKVQuantizer: the reference's context-manager surface over a cache tuple."""
    from fastcache_amd.presses import ImprovedKVQuantizer, SimpleKVQuantizer, press_select
    from oracle import presses as op
    g = torch.Generator().manual_seed(2)
    pkv = tuple((torch.randn(1, 4, 50, 128, generator=g).bfloat16(), torch.randn(1, 4, 50, 128, generator=g).bfloat16())
                for _ in range(3))
    dev_pkv = tuple((k.to(dev), v.to(dev)) for k, v in pkv)
    qz = press_select("Quantized")
    assert isinstance(qz, SimpleKVQuantizer) and qz.nbits == 4
    with qz(None) as q:
        out = q.quantize_cache(dev_pkv)
    for (k, v), (qk, qv) in zip(pkv, out):
        assert torch.equal(qk.cpu(), op.fake_quantize(k, 4, True)[0]) and torch.equal(qv.cpu(), op.fake_quantize(v, 4, True)[0])
    iq = ImprovedKVQuantizer(nbits=8)
    out = iq.quantize_cache(dev_pkv)
    for i, ((k, v), (qk, qv)) in enumerate(zip(pkv, out)):
        rk, rs, rm = op.fake_quantize(k, 8, False)
        assert torch.equal(qk.cpu(), rk) and torch.equal(iq.cache[f"k_{i}"]["scale"].cpu(), rs)
        assert torch.equal(iq.cache[f"k_{i}"]["max_val"].cpu(), rm)
    deq = iq.dequantize_cache(out)
    assert torch.equal(deq[0][0].cpu(), out[0][0].cpu() * iq.cache["k_0"]["scale"].cpu())


@pytest.mark.parametrize("shape,bits", [((1, 100), 2), ((3, 5, 7), 16), ((2, 1), 4), ((4, 1000), 3)])
def test_fake_quantize_odd_shapes(dev, shape, bits):
    """Rows that are no multiple of the wavefront, one-element rows, the smallest and the widest code range."""
    from oracle import presses as op
    g = torch.Generator().manual_seed(sum(shape) + bits)
    x = torch.randn(*shape, generator=g)
    for per_tensor in (False, True):
        ref = op.fake_quantize(x, bits, per_tensor)[0]
        got = ops.fake_quantize(x.to(dev), bits, per_tensor).cpu()
        assert torch.equal(torch.nan_to_num(got, nan=-7.0), torch.nan_to_num(ref, nan=-7.0)), per_tensor


def test_kvpress_method_adapter(dev):
    """KVPressMethod: a press by name, called on bare tensors; every name of the reference's table resolves, the
    results equal the press called directly, unknown names raise as there."""
    from fastcache_amd import presses
    g = torch.Generator().manual_seed(9)
    k = torch.randn(2, 2, 300, 128, generator=g).half().to(dev)
    v = torch.randn(2, 2, 300, 128, generator=g).half().to(dev)
    q = torch.randn(2, 8, 64, 128, generator=g).half().to(dev)
    m = ac.KVPressMethod("SnapKV", compression_ratio=0.5, window_size=64, kernel_size=7)
    assert m.name == "kvpress_snapkv"
    ck, cv = m.compress(k, v, queries=q)
    rk, rv = presses.SnapKVPress(compression_ratio=0.5, window_size=64, kernel_size=7).compress(None, None, k, v, None, {"queries": q})
    assert ck.shape == (2, 2, 150, 128) and torch.equal(ck, rk) and torch.equal(cv, rv)
    ck, cv = ac.KVPressMethod("knorm", 0.25).compress(k, v)
    assert ck.shape == (2, 2, 225, 128)
    tk, _ = ac.KVPressMethod("think", 0.5, window_size=32).compress(k.clone(), v, queries=q[:, :, -32:])
    assert int((tk == 0).all(dim=2).sum()) == 2 * 2 * 64
    sk, _ = ac.KVPressMethod("simlayer", 0.5, lazy_threshold=0.0, n_recent=100).compress(k, v, queries=q[:, :, -1:])
    assert sk.shape == (2, 2, 4 + 99, 128)
    for name in ("streaming_llm", "observed_attention", "expected_attention", "tova", "random"):
        assert ac.KVPressMethod(name, 0.3).press.compression_ratio == 0.3
    with pytest.raises(ValueError):
        ac.KVPressMethod("h2o").compress(k, v)


def test_mlp_method_adapter_and_registry(dev):
    """``get_method('mlp', compressor=...)``: one layer's K and V (with ``layer_idx``) and all layers at once against
    the oracle's MLP compressor; the registry resolves every family of names, caches instances and rejects others."""
    from types import SimpleNamespace
    from fastcache_amd.kernels import BatchedGEMMCompressor
    from fastcache_amd.utils_ccm import KVCacheLinearDecoupleCompressor
    dtype, L, B, H, S, cf = torch.float16, 3, 2, 2, 90, 2
    cfg = SimpleNamespace(text_config=SimpleNamespace(num_hidden_layers=L, num_key_value_heads=H, hidden_size=H * 128,
                                                      head_dim=128, num_attention_heads=H))
    torch.manual_seed(11)
    orig = KVCacheLinearDecoupleCompressor(cfg, compression_factor=cf).to(dev).to(dtype).eval()
    sd = occm.reference_init_state_dict("linear_decouple", L, 128, cf, seed=11)
    bat = BatchedGEMMCompressor(num_layers=L, num_heads=H, head_dim=128, compression_factor=cf)
    bat.load_from_original_compressor(orig)
    g = torch.Generator().manual_seed(3)
    k = torch.randn(L, B, H, S, 128, generator=g).to(dtype)
    v = torch.randn(L, B, H, S, 128, generator=g).to(dtype)
    it_len = [50, 40]
    ref = occm.linear_decouple_forward([(k[l], v[l]) for l in range(L)], it_len, sd, cf, 1)
    m = ac.get_method("mlp", compressor=bat)
    assert m.name == "mlp_compress" and ac.get_method("mlp", compressor=bat) is m
    ck, cv = m.compress(k[1].to(dev), v[1].to(dev), it_len=it_len, layer_idx=1)
    assert ck.shape == (B, H, 45, 128)
    assert_mlp_close(ck.cpu(), ref[1][0], dtype)
    assert_mlp_close(cv.cpu(), ref[1][1], dtype)
    ak, av = ac.get_method("mlp_compress", compressor=orig).compress(k.to(dev), v.to(dev), it_len=it_len)
    assert ak.shape == (L, B, H, 45, 128) and torch.equal(ak[1], ck) and torch.equal(av[1], cv)
    for l in range(L):
        assert_mlp_close(ak[l].cpu(), ref[l][0], dtype)
    with pytest.raises(RuntimeError, match="not initialized"):
        ac.MLPCompressionMethod().compress(k[0].to(dev), v[0].to(dev))
    # the other families of names
    assert isinstance(ac.get_method("kvpress_snapkv", compression_ratio=0.5), ac.KVPressMethod)
    assert isinstance(ac.get_method("knorm"), ac.KVPressMethod) and ac.get_method("knorm").name == "kvpress_knorm"
    assert ac.get_method("quant_nf4").name == "quant_nf4" and ac.get_method("int8").name == "quant_int8"
    assert {"mlp", "kvpress_snapkv", "quant_int4"} <= set(ac.list_methods())
    ac.MethodRegistry.register("mine", ac.MLPCompressionMethod)
    assert "mine" in ac.list_methods() and isinstance(ac.get_method("mine"), ac.MLPCompressionMethod)
    with pytest.raises(ValueError, match="Unknown compression method"):
        ac.get_method("zip")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [128, 64, 256, 40])
def test_quantisers_special_rows_all_row_lengths(dev, dtype, d):
    """Rows of 128 / 256 / 512 bytes take the 16-bytes-per-lane kernels, other lengths the generic ones: both against
    the eager expressions bit for bit, on random rows plus an all-zero row, a row with a NaN, a row with an infinity,
    a constant row, a one-hot row and a row of tiny values; row counts that leave the last block partly empty."""
    g = torch.Generator().manual_seed(d)
    x = (torch.randn(37, d, generator=g) * 3).to(dtype)
    x[1] = 0
    x[2, 5] = float("nan")
    x[3, 7] = float("inf")
    x[4] = -1.75
    x[5] = 0
    x[5, d - 1] = 2.5
    x[6] = x[6] * 1e-6
    xd = x.to(dev)

    def same(a, b):
        a, b = a.cpu(), b
        assert a.dtype == b.dtype and a.shape == b.shape
        if a.is_floating_point():
            assert torch.equal(a.isnan(), b.isnan()) and torch.equal(a.nan_to_num(7.0), b.nan_to_num(7.0))
        else:
            assert torch.equal(a, b)

    q, s = ops.quantize_rows(xd, 8)
    rq, rs = oa.quantize_int8(x)
    same(s, rs)
    same(q, rq)                                  # NaN quotients (NaN row, 0/0 of a zero row in fp16, inf/inf) give code 0
    ok_rows = ~x.isnan().any(-1)
    q, p = ops.quantize_rows_asym(xd)
    rq, rp = oa.quantize_int8_asymmetric(x)
    ok_asym = ok_rows & ~x.isinf().any(-1)       # inf - inf inside the row gives NaN codes
    assert torch.equal(q.cpu()[ok_asym], rq[ok_asym])
    same(p[..., 0], rp[..., 0])
    assert bool((p.cpu()[..., 1].float().nan_to_num(-1) == rp[..., 1].float().nan_to_num(-1)).all())
    if d % 8 == 0:
        for nf4 in (False, True):
            q, s = ops.quantize_group4(xd, d, nf4)
            rq, rs = (oa.quantize_nf4 if nf4 else oa.quantize_int4)(x, d)
            same(s, rs)
            same(q, rq)                          # NaN quotients: integer 0 + 8 (int4), first level (nf4)
    for bits in (4, 8):
        y, sc, mx = ops.fake_quantize(xd, bits, per_tensor=False, return_params=True)
        qmax = 2 ** (bits - 1) - 1
        rmx = x.abs().amax(dim=-1, keepdim=True)
        rsc = rmx / qmax
        ry = (x / rsc).round().clamp(-qmax - 1, qmax) * rsc
        same(mx, rmx)
        same(sc, rsc)
        same(y, ry)
