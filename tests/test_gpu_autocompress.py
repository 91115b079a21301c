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
    with pytest.raises(FastcacheError):
        ac.QuantizationMethod("fp8").compress(X.to(dev), V.to(dev))


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
