"""GPU parity of the fp32 ("train / eval") recurrence, through the C-ABI entry adkv_quant_f32 and
its host-side mirrors, against the CPU oracle: integer codes, dequantised values and fp32 state
must be bit-identical."""
import math

import numpy as np
import pytest
import torch

from adkv_amd import synth

pytestmark = pytest.mark.gpu


def _params(C, seed, bits):
    g = torch.Generator().manual_seed(seed)
    qu = 2 ** (bits - 1) - 1
    return dict(
        zp=0.3 * torch.randn(C, generator=g),
        sc=0.5 + torch.rand(C, generator=g),
        alpha=0.9 + 0.099 * torch.rand(C, generator=g),
        beta=0.05 * torch.rand(C, generator=g),
        tgt=torch.full((C,), qu / 2.0))


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int32)


@pytest.mark.parametrize("B,T,C,bits", [(1, 1, 64, 4), (2, 37, 100, 4), (3, 257, 130, 2), (1, 64, 512, 8),
                                        (1, 1024, 4096, 4)])
def test_quant_f32_bit_exact(gpu, oracle, B, T, C, bits):
    from adkv_amd.train import quant_f32
    p = _params(C, 7 + T, bits)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(B, T, C, generator=g) * 2.0
    x[:, :, ::17] += 6.0 * torch.sin(0.02 * torch.arange(T, dtype=torch.float32))[None, :, None]
    ql, qu = -2 ** (bits - 1), 2 ** (bits - 1) - 1
    want = oracle.quant_f32(x.numpy(), *[p[k].numpy() for k in ("zp", "sc", "alpha", "beta", "tgt")],
                            bits=bits, want_seq=True)
    zp = torch.empty(B, C, device=gpu)
    sc = torch.empty(B, C, device=gpu)
    xhat, codes, zs, ss = quant_f32(
        x.to(gpu), p["alpha"].to(gpu), p["beta"].to(gpu), p["tgt"].to(gpu), ql, qu,
        math.exp(-4.0), math.exp(4.0), zp_state=zp, sc_state=sc,
        zp_init=p["zp"].to(gpu), sc_init=p["sc"].to(gpu), want_codes=True, output_states=True)
    torch.cuda.synchronize()
    assert np.array_equal(codes.cpu().numpy(), want["codes"])
    for got, key in ((xhat, "xhat"), (zp, "zp"), (sc, "sc"), (zs, "zp_seq"), (ss, "sc_seq")):
        assert np.array_equal(_bits(got).numpy(), want[key].view(np.int32)), key


def _run_no_seq(gpu, x, p, bits, dtype=torch.float32):
    from adkv_amd.train import quant_f32
    B, T, C = x.shape
    ql, qu = -2 ** (bits - 1), 2 ** (bits - 1) - 1
    zp = torch.empty(B, C, device=gpu)
    sc = torch.empty(B, C, device=gpu)
    xhat, codes, _, _ = quant_f32(
        x.to(dtype).to(gpu), p["alpha"].to(gpu), p["beta"].to(gpu), p["tgt"].to(gpu), ql, qu,
        math.exp(-4.0), math.exp(4.0), zp_state=zp, sc_state=sc,
        zp_init=p["zp"].to(gpu), sc_init=p["sc"].to(gpu), want_codes=True)
    torch.cuda.synchronize()
    return xhat, codes, zp, sc


def _same_bits_or_both_nan(got, want):
    g, w = got.detach().cpu().float().numpy(), np.asarray(want, dtype=np.float32)
    both_nan = np.isnan(g) & np.isnan(w)
    return np.array_equal(np.where(both_nan, 0, g.view(np.int32)), np.where(both_nan, 0, w.view(np.int32)))


@pytest.mark.parametrize("B,T,C,bits", [(1, 7, 64, 4), (2, 8, 100, 4), (2, 37, 100, 4), (3, 257, 130, 2),
                                        (1, 100, 512, 8), (1, 1024, 4096, 4)])
def test_quant_f32_without_state_sequence_bit_exact(gpu, oracle, B, T, C, bits):
    """The production form (no state sequence recorded) runs groups of 8 tokens speculatively and
    repeats the ones that came near a rounding boundary: same codes, values and state as the oracle."""
    p = _params(C, 7 + T, bits)
    g = torch.Generator().manual_seed(T)
    x = torch.randn(B, T, C, generator=g) * 2.0
    x[:, :, ::17] += 6.0 * torch.sin(0.02 * torch.arange(T, dtype=torch.float32))[None, :, None]
    want = oracle.quant_f32(x.numpy(), *[p[k].numpy() for k in ("zp", "sc", "alpha", "beta", "tgt")], bits=bits)
    xhat, codes, zp, sc = _run_no_seq(gpu, x, p, bits)
    assert np.array_equal(codes.cpu().numpy(), want["codes"])
    for got, key in ((xhat, "xhat"), (zp, "zp"), (sc, "sc")):
        assert np.array_equal(_bits(got).numpy(), want[key].view(np.int32)), key


def test_quant_f32_rounding_boundaries_and_non_finite_inputs(gpu, oracle):
    """First tokens placed on rounding boundaries (x - zp = (k + 1/2) * sc and its fp32 neighbours),
    and NaN / infinite / huge inputs scattered over the stream: the speculative path has to notice
    all of them and fall back; NaN handling follows torch.clamp (NaN stays NaN, its code is 0)."""
    B, T, C, bits = 2, 64, 256, 4
    p = _params(C, 11, bits)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, T, C, generator=g) * 2.0
    k = torch.arange(C, dtype=torch.float32) % 16 - 8.0
    tie = p["zp"] + (k + 0.5) * p["sc"]
    x[0, 0] = tie
    x[1, 0] = torch.nextafter(tie, torch.full_like(tie, 1e9))
    x[1, 8] = torch.nextafter(x[1, 8], torch.full_like(tie, -1e9))
    x[0, 5, 3] = float("nan")
    x[0, 17, 40] = float("inf")
    x[1, 30, 41] = float("-inf")
    x[1, 9, 100] = 3.0e38
    x[0, 33, 101] = -1.0e30
    want = oracle.quant_f32(x.numpy(), *[p[k].numpy() for k in ("zp", "sc", "alpha", "beta", "tgt")], bits=bits)
    xhat, codes, zp, sc = _run_no_seq(gpu, x, p, bits)
    assert np.array_equal(codes.cpu().numpy(), want["codes"])
    assert _same_bits_or_both_nan(xhat, want["xhat"])
    assert _same_bits_or_both_nan(zp, want["zp"])
    assert _same_bits_or_both_nan(sc, want["sc"])
    assert np.isnan(want["zp"]).any()            # the NaN really reached the state of its channel


@pytest.mark.parametrize("dtype,C", [(torch.float16, 130), (torch.bfloat16, 129), (torch.float16, 65)])
def test_quant_f32_half_inputs_odd_and_even_widths(gpu, oracle, dtype, C):
    """16-bit inputs take aligned 32-bit loads when rows allow it (even C) and plain 16-bit loads
    otherwise (odd C): both give the oracle's result on the values as read."""
    B, T = 2, 50
    p = _params(C, 3, 4)
    x = (torch.randn(B, T, C, generator=torch.Generator().manual_seed(C)) * 1.5).to(dtype)
    want = oracle.quant_f32(x.float().numpy(), *[p[k].numpy() for k in ("zp", "sc", "alpha", "beta", "tgt")])
    xhat, codes, zp, sc = _run_no_seq(gpu, x.float(), p, 4, dtype=dtype)
    assert np.array_equal(codes.cpu().numpy(), want["codes"])
    assert torch.equal(xhat.cpu(), torch.from_numpy(want["xhat"]).to(dtype))
    assert np.array_equal(_bits(zp).numpy(), want["zp"].view(np.int32))
    assert np.array_equal(_bits(sc).numpy(), want["sc"].view(np.int32))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quant_f32_half_inputs_in_place_and_chunked(gpu, oracle, dtype):
    """16-bit buffers are read up to fp32 and written back rounded (as the reference's Triton kernel
    does on a 16-bit cache); walking the stream in three calls with the carried state equals one."""
    from adkv_amd.train import quant_f32
    B, T, C = 2, 96, 192
    p = _params(C, 5, 4)
    x = (torch.randn(B, T, C, generator=torch.Generator().manual_seed(9)) * 1.5).to(dtype)
    want = oracle.quant_f32(x.float().numpy(), *[p[k].numpy() for k in ("zp", "sc", "alpha", "beta", "tgt")])
    buf = torch.zeros(B, 128, C, dtype=dtype, device=gpu)   # strided view of a larger buffer
    buf[:, :T] = x.to(gpu)
    zp = p["zp"].repeat(B, 1).to(gpu).contiguous()
    sc = p["sc"].repeat(B, 1).to(gpu).contiguous()
    for a, b in ((0, 1), (1, 40), (40, T)):
        v = buf[:, a:b]
        quant_f32(v, p["alpha"].to(gpu), p["beta"].to(gpu), p["tgt"].to(gpu), -8, 7,
                  math.exp(-4.0), math.exp(4.0), zp_state=zp, sc_state=sc, out=v)
    torch.cuda.synchronize()
    assert torch.equal(buf[:, :T].cpu(), torch.from_numpy(want["xhat"]).to(dtype))
    assert np.array_equal(_bits(zp).numpy(), want["zp"].view(np.int32))
    assert np.array_equal(_bits(sc).numpy(), want["sc"].view(np.int32))
    assert torch.count_nonzero(buf[:, T:]) == 0


def test_train_model_forward_and_chunk_forward(gpu, oracle):
    from adkv_amd.train import ADKVTrainModel, adkv_chunk_forward
    torch.manual_seed(3)
    C, B, T = 256, 2, 70
    m = ADKVTrainModel(C, bits=4).to(gpu)
    with torch.no_grad():
        m.alpha.normal_(2.0, 0.5)
        m.beta.normal_(0.0, 1.0)
        m.init_zp.normal_(0.0, 0.2)
        m.init_log_sc.normal_(0.0, 0.2)
    x = torch.randn(B, T, C)
    out, zs, ss = m(x.to(gpu), output_states=True)
    al, be = m.get_alpha().detach().cpu(), m.get_beta().detach().cpu()
    want = oracle.quant_f32(x.numpy(), m.init_zp.detach().cpu().numpy(), m.get_sc().detach().cpu().numpy(),
                            al.numpy(), be.numpy(), m.target.detach().cpu().numpy(), want_seq=True)
    assert np.array_equal(_bits(out).numpy(), want["xhat"].view(np.int32))
    assert np.array_equal(_bits(zs).numpy(), want["zp_seq"].view(np.int32))
    assert np.array_equal(_bits(ss).numpy(), want["sc_seq"].view(np.int32))
    # the chunk function: state in -> state out, arguments untouched
    zp0 = m.init_zp.detach().expand(B, -1).contiguous()
    sc0 = m.get_sc().detach().expand(B, -1).contiguous()
    keep = zp0.clone()
    o1, zp1, sc1, _, _ = adkv_chunk_forward(x[:, :32].to(gpu), zp0, sc0, al.to(gpu), be.to(gpu),
                                            m.target.detach(), 7, -8, m.sc_min, m.sc_max, False)
    o2, zp2, sc2, _, _ = adkv_chunk_forward(x[:, 32:].to(gpu), zp1, sc1, al.to(gpu), be.to(gpu),
                                            m.target.detach(), 7, -8, m.sc_min, m.sc_max, False)
    assert torch.equal(zp0, keep)
    assert np.array_equal(_bits(torch.cat([o1, o2], 1)).numpy(), want["xhat"].view(np.int32))
    assert np.array_equal(_bits(zp2).numpy(), want["zp"].view(np.int32))
    assert np.array_equal(_bits(sc2).numpy(), want["sc"].view(np.int32))


def test_eval_cache_update_matches_oracle(gpu, oracle):
    """The eval cache quantises on write with persistent state: prefill of 150 tokens, then five
    single-token updates, equals the oracle over the whole stream."""
    from adkv_amd.hf.llama_adkv_eval import KVCacheLayer_ADKV
    B, C, T = 2, 128, 155
    pk, pv = _params(C, 1, 4), _params(C, 2, 4)
    g = torch.Generator().manual_seed(4)
    k, v = torch.randn(B, T, C, generator=g), torch.randn(B, T, C, generator=g)
    layer = KVCacheLayer_ADKV()
    args = [pk[n].to(gpu) for n in ("zp", "sc", "alpha", "beta", "tgt")] + \
           [pv[n].to(gpu) for n in ("zp", "sc", "alpha", "beta", "tgt")]
    cuts = [0, 150, 151, 152, 153, 154, 155]
    for a, b in zip(cuts[:-1], cuts[1:]):
        ks, vs = layer.update(k[:, a:b].to(gpu), v[:, a:b].to(gpu), *args)
        assert ks.shape == (B, b, C) and layer.get_seq_length() == b
    wk = oracle.quant_f32(k.numpy(), *[pk[n].numpy() for n in ("zp", "sc", "alpha", "beta", "tgt")])
    wv = oracle.quant_f32(v.numpy(), *[pv[n].numpy() for n in ("zp", "sc", "alpha", "beta", "tgt")])
    assert np.array_equal(_bits(ks).numpy(), wk["xhat"].view(np.int32))
    assert np.array_equal(_bits(vs).numpy(), wv["xhat"].view(np.int32))
    assert np.array_equal(_bits(layer.key_scale).numpy(), wk["sc"].view(np.int32))
    assert np.array_equal(_bits(layer.value_dc).numpy(), wv["zp"].view(np.int32))


def test_cfg1_fp16_deployment_tracks_fp32_quantiser(gpu, oracle):
    """Config 1 (one sequence, 32 heads x 128 channels, 1024 tokens, K with outlier channels):
    the fp16 deployment recurrence through the drop-in and the fp32 recurrence are different
    arithmetic over a feedback loop that amplifies a one-step difference, so their code streams
    are not comparable element by element.  What must hold is that both reconstruct the input
    equally well: the RMS errors agree within 5 % and the two reconstructions differ by no more
    than quantisation noise."""
    from adkv_amd.kernel import gemv
    B, H, D, T = 1, 32, 128, 1024
    p = synth.make_params(H, D, seed=3)
    x = synth.make_k(B, H, T, D, dtype=torch.float32).half()          # [B, H, T, D]
    cache = synth.alloc_cache(B, H, T, D, gpu)
    gemv.encode_kv(cache, x.to(gpu), *[t.to(gpu) for t in p.astuple()], math.exp(-4.0), math.exp(4.0))
    torch.cuda.synchronize()
    pn = [t.numpy() for t in p.astuple()]
    xhat_b, _ = oracle.replay_f16(cache.cpu().numpy(), *pn, T)
    xa = x.float().permute(0, 2, 1, 3).reshape(B, T, H * D)
    want = oracle.quant_f32(xa.numpy(), *[t.float().reshape(-1).numpy() for t in p.astuple()])
    xhat_a = want["xhat"].reshape(B, T, H, D).transpose(0, 2, 1, 3)
    xn = x.float().numpy()
    # the first tokens are the filter's transient from (zp_init, scale_init); compare after it
    w = slice(64, None)
    rms = lambda a: float(np.sqrt(np.mean(np.square(a, dtype=np.float64))))
    ea, eb = rms(xhat_a[:, :, w] - xn[:, :, w]), rms(xhat_b.astype(np.float32)[:, :, w] - xn[:, :, w])
    assert abs(ea - eb) <= 0.05 * ea, (ea, eb)
    assert rms(xhat_a[:, :, w] - xhat_b.astype(np.float32)[:, :, w]) <= 1.5 * ea
