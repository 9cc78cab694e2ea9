"""Every row / attention / GEMM entry point of the C-ABI on operands that live inside larger buffers:
rows at a pitch (aligned and unaligned), ragged sizes, outputs surrounded by a byte pattern that must
survive the call, inputs surrounded by bytes that decode to NaN (floating point) or -1 (integers), so that
a read of a gap that reaches a result shows up as a mismatch.  The expected values come from the same
entry points on contiguous copies, which the parity tests compare with the oracle."""

import numpy as np
import pytest
import torch

from tests.util import DEV, rng

pytestmark = pytest.mark.gpu

OUT_FILL, IN_FILL, PAD = 0x5A, 0xFF, 4096


def _lib():
    from triton_int_amd import _lib as L
    return L


class Held:
    """A [rows, cols] view with `pitch` elements between rows, `lead` elements into a byte buffer that is
    filled with `fill` (leading offset: lets a test choose the alignment of the first element)."""

    def __init__(self, rows, cols, dtype, pitch=None, fill=OUT_FILL, lead=0, data=None):
        self.rows, self.cols, self.dtype = rows, cols, dtype
        self.pitch = cols if pitch is None else pitch
        self.esz = torch.empty((), dtype=dtype).element_size()
        self.lead = lead
        self.fill = fill
        nbytes = (lead + max(rows, 1) * self.pitch) * self.esz
        self.buf = torch.full((PAD + nbytes + PAD,), fill, dtype=torch.uint8, device=DEV)
        body = self.buf[PAD:PAD + nbytes].view(dtype)[lead:]
        self.view = body.view(max(rows, 1), self.pitch)[:rows, :cols]
        if data is not None:
            self.view.copy_(data.to(DEV))

    @property
    def ptr(self):
        return self.view.data_ptr() if self.view.numel() else self.buf.data_ptr() + PAD + self.lead * self.esz

    def surroundings_intact(self):
        """True when every byte outside the view still holds the fill pattern."""
        b = self.buf.cpu().numpy().copy()
        for r in range(self.rows):
            o = PAD + (self.lead + r * self.pitch) * self.esz
            b[o:o + self.cols * self.esz] = self.fill
        return bool((b == self.fill).all())


def _stream():
    return _lib().current_stream(torch.device(DEV))


def _ok(rc, what):
    _lib().check(rc, what)
    torch.cuda.synchronize()


def _f32(g, *shape):
    return torch.from_numpy(g.standard_normal(shape).astype(np.float32))


def _i8(g, *shape, lo=-127, hi=127):
    return torch.from_numpy(g.integers(lo, hi + 1, size=shape, dtype=np.int8))


ROW_SHAPES = [(7, 1001, 1003, 1), (5, 1024, 1040, 0), (3, 5120, 5124, 4), (9, 300, 300, 0), (4, 7, 16, 3), (2, 8193, 8200, 0),
              (6, 20480, 20484, 0), (1, 33, 40, 0)]


@pytest.mark.parametrize("rows,cols,pitch,lead", ROW_SHAPES)
def test_layernorm_q_and_dq_add_layernorm_q_stay_inside_their_rows(rows, cols, pitch, lead):
    L = _lib()
    from triton_int_amd.kernels import fused
    g = rng(rows * 31 + cols)
    x, gamma, beta = _f32(g, rows, cols), _f32(g, cols) * 2 + 20, _f32(g, cols) * 2
    hx = Held(rows, cols, torch.float32, pitch, IN_FILL, lead, x)
    hy = Held(rows, cols, torch.int8, pitch + 5, OUT_FILL, lead)
    hmean, hrstd = Held(1, rows, torch.float32), Held(1, rows, torch.float32)
    gg, gb = Held(1, cols, torch.float32, None, IN_FILL, lead, gamma[None]), Held(1, cols, torch.float32, None, IN_FILL, lead, beta[None])
    print(f"ti_layernorm_q rows={rows} cols={cols} pitch={pitch} lead={lead}", flush=True)
    _ok(L.lib().ti_layernorm_q(hx.ptr, hx.pitch, gg.ptr, gb.ptr, 1e-5, hy.ptr, hy.pitch, rows, cols, 0, L.ROUND_RNE_CLAMP,
                               hmean.ptr, hrstd.ptr, _stream()), "ti_layernorm_q")
    want, wmean, wrstd = fused.layer_norm_fwd_fused_single_pass_q(x.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5, _return_stats=True)
    assert hy.surroundings_intact() and hmean.surroundings_intact() and hrstd.surroundings_intact()
    assert (hy.view.int() - want.int()).abs().max().item() <= 1
    assert torch.allclose(hmean.view[0], wmean, rtol=0, atol=1e-4) and torch.allclose(hrstd.view[0], wrstd, rtol=1e-4, atol=0)

    acc = torch.from_numpy(g.integers(-2**20, 2**20 + 1, size=(rows, cols), dtype=np.int32))
    hacc = Held(rows, cols, torch.int32, pitch + 4, IN_FILL, lead, acc)
    hro = Held(rows, cols, torch.float32, pitch + 8, OUT_FILL, lead)
    hy = Held(rows, cols, torch.int8, pitch + 16, OUT_FILL, lead)
    print(f"ti_dq_add_layernorm_q rows={rows} cols={cols} pitch={pitch} lead={lead}", flush=True)
    _ok(L.lib().ti_dq_add_layernorm_q(hacc.ptr, hacc.pitch, 1e-5, None, hx.ptr, hx.pitch, gg.ptr, gb.ptr, 1e-5, hro.ptr, hro.pitch,
                                      hy.ptr, hy.pitch, None, 0, rows, cols, L.ROUND_RNE_CLAMP, None, None, _stream()),
        "ti_dq_add_layernorm_q")
    wres, wy = fused.dq_add_layernorm_q(acc.to(DEV), 1e-5, x.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
    assert hro.surroundings_intact() and hy.surroundings_intact()
    assert torch.equal(hro.view, wres) and (hy.view.int() - wy.int()).abs().max().item() <= 1


@pytest.mark.parametrize("rows,cols,pitch,lead", ROW_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_layernorm_fp_stays_inside_its_rows(rows, cols, pitch, lead, dtype):
    L = _lib()
    from triton_int_amd.kernels import fused
    g = rng(rows * 37 + cols)
    x, skip = _f32(g, rows, cols).to(dtype), _f32(g, rows, cols).to(dtype)
    gamma, beta = (_f32(g, cols) * 0.1 + 1).to(dtype), (_f32(g, cols) * 0.1).to(dtype)
    hx, hs = Held(rows, cols, dtype, pitch, IN_FILL, lead, x), Held(rows, cols, dtype, pitch + 8, IN_FILL, lead, skip)
    ho, hso = Held(rows, cols, dtype, pitch + 3, OUT_FILL, lead), Held(rows, cols, dtype, pitch, OUT_FILL, lead)
    gg, gb = Held(1, cols, dtype, None, IN_FILL, lead, gamma[None]), Held(1, cols, dtype, None, IN_FILL, lead, beta[None])
    print(f"ti_layernorm_fp {dtype} rows={rows} cols={cols} pitch={pitch} lead={lead}", flush=True)
    _ok(L.lib().ti_layernorm_fp(hx.ptr, hx.pitch, hs.ptr, hs.pitch, L.TORCH_TO_DT[dtype], gg.ptr, gb.ptr, 1e-5, 0, ho.ptr, ho.pitch,
                                hso.ptr, hso.pitch, rows, cols, _stream()), "ti_layernorm_fp")
    want, want_skip = fused.skip_layer_norm_fwd_fused_single_pass2(x.to(DEV), skip.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5)
    assert ho.surroundings_intact() and hso.surroundings_intact()
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    assert torch.allclose(ho.view.float(), want.float(), **tol) and torch.allclose(hso.view.float(), want_skip.float(), **tol)
    assert not torch.isnan(ho.view.float()).any()


@pytest.mark.parametrize("rows,cols,pitch,lead", ROW_SHAPES + [(12, 1536, 1552, 0), (5, 2048, 2051, 2)])
def test_softmax_q_and_quantize_per_token_stay_inside_their_rows(rows, cols, pitch, lead):
    L = _lib()
    from triton_int_amd.kernels import fused
    g = rng(rows * 41 + cols)
    if cols <= 8192:
        x = _i8(g, rows, cols, lo=-128)
        hx, hy = Held(rows, cols, torch.int8, pitch, IN_FILL, lead, x), Held(rows, cols, torch.int8, pitch + 1, OUT_FILL, lead)
        print(f"ti_softmax_q rows={rows} cols={cols} pitch={pitch} lead={lead}", flush=True)
        _ok(L.lib().ti_softmax_q(hx.ptr, hx.pitch, 0.05, hy.ptr, hy.pitch, rows, cols, 0, _stream()), "ti_softmax_q")
        assert hy.surroundings_intact() and torch.equal(hy.view, fused.softmax_q(x.to(DEV), 0.05))
    for dtype in (torch.float32, torch.float16):
        t = (_f32(g, rows, cols) * 3).to(dtype)
        ht = Held(rows, cols, dtype, pitch, IN_FILL, lead, t)
        hq, hs = Held(rows, cols, torch.int8, pitch + 4, OUT_FILL, lead), Held(1, rows, dtype)
        print(f"ti_quantize_per_token_absmax {dtype} rows={rows} cols={cols} pitch={pitch} lead={lead}", flush=True)
        _ok(L.lib().ti_quantize_per_token_absmax(ht.ptr, L.TORCH_TO_DT[dtype], ht.pitch, hq.ptr, hq.pitch, hs.ptr, rows, cols, _stream()),
            "ti_quantize_per_token_absmax")
        wq, ws = fused.quantize_per_token_absmax(t.to(DEV))
        assert hq.surroundings_intact() and hs.surroundings_intact()
        assert torch.equal(hq.view, wq) and torch.equal(hs.view[0], ws.view(-1))


@pytest.mark.parametrize("n,lead", [(1, 0), (3, 1), (1000, 0), (4099, 3), (16384 + 5, 4), (1 << 20, 0)])
def test_gelu_q_stays_inside_its_range(n, lead):
    L = _lib()
    from triton_int_amd.kernels import fused
    g = rng(n)
    x = _f32(g, 1, n) * 3
    hx, hy = Held(1, n, torch.float32, None, IN_FILL, lead, x), Held(1, n, torch.int8, None, OUT_FILL, lead)
    s = torch.tensor([20.0], device=DEV)
    print(f"ti_gelu_q n={n} lead={lead}", flush=True)
    _ok(L.lib().ti_gelu_q(hx.ptr, s.data_ptr(), hy.ptr, n, L.ROUND_RNE_CLAMP, _stream()), "ti_gelu_q")
    assert hy.surroundings_intact() and torch.equal(hy.view[0], fused.gelu_q(x[0].to(DEV), 20.0))


@pytest.mark.parametrize("rows,cols,spitch,dpitch,lead", [(70, 33, 40, 75, 0), (129, 257, 257, 129, 1), (64, 64, 80, 64, 0),
                                                          (16, 5120, 5120, 2048, 0), (5, 1, 3, 9, 2), (200, 48, 64, 208, 0)])
def test_transpose_and_kv_append_stay_inside_their_views(rows, cols, spitch, dpitch, lead):
    L = _lib()
    g = rng(rows * 43 + cols)
    x = _i8(g, rows, cols, lo=-128)
    hx, hd = Held(rows, cols, torch.int8, spitch, IN_FILL, lead, x), Held(cols, rows, torch.int8, dpitch, OUT_FILL, lead)
    print(f"ti_transpose_i8 rows={rows} cols={cols} spitch={spitch} dpitch={dpitch} lead={lead}", flush=True)
    _ok(L.lib().ti_transpose_i8(hx.ptr, hx.pitch, hd.ptr, hd.pitch, rows, cols, _stream()), "ti_transpose_i8")
    assert hd.surroundings_intact() and torch.equal(hd.view.cpu(), x.t().contiguous())


@pytest.mark.parametrize("S,heads,D,T", [(16, 5, 128, 300), (48, 3, 64, 100), (1, 2, 16, 5), (70, 2, 128, 70)])
def test_kv_append_writes_only_the_new_positions(S, heads, D, T):
    L = _lib()
    g = rng(S * 47 + heads)
    H = heads * D
    k_new, v_new = _i8(g, S, H, lo=-128), _i8(g, S, H, lo=-128)
    hk, hv = Held(S, H, torch.int8, H + 16, IN_FILL, 0, k_new), Held(S, H, torch.int8, 3 * H, IN_FILL, 0, v_new)
    # caches as guarded buffers: K [heads, T, D] (rows = heads * T), V^T [heads * D, T]; positions T-S .. T-1 are written
    hkc, hvc = Held(heads * T, D, torch.int8, None, OUT_FILL), Held(H, T, torch.int8, T + 7, OUT_FILL)
    k_dst = hkc.ptr + (T - S) * D
    vt_dst = hvc.ptr + (T - S)
    print(f"ti_kv_append_i8 S={S} heads={heads} D={D} T={T}", flush=True)
    _ok(L.lib().ti_kv_append_i8(hk.ptr, hk.pitch, hv.ptr, hv.pitch, k_dst, T * D, vt_dst, hvc.pitch, S, heads, D, _stream()),
        "ti_kv_append_i8")
    kc = hkc.view.view(heads, T, D).cpu()
    assert torch.equal(kc[:, T - S:], k_new.view(S, heads, D).permute(1, 0, 2))
    assert (kc[:, :T - S] == OUT_FILL).all() and hkc.surroundings_intact()
    vc = hvc.view.cpu()
    assert torch.equal(vc[:, T - S:], v_new.t().contiguous()) and (vc[:, :T - S] == OUT_FILL).all() and hvc.surroundings_intact()


@pytest.mark.parametrize("BH,S,T,q_len", [(2, 200, 336, 0), (3, 5, 80, 5), (2, 48, 272, 48), (1, 16, 2048, 16), (2, 144, 144, 144), (1, 1, 16, 0)])
def test_attention_i8_stays_inside_its_views(BH, S, T, q_len):
    L = _lib()
    from triton_int_amd.kernels import fused
    D = 128
    g = rng(BH * 53 + S + T)
    q, k, vt = _i8(g, BH * S, D), _i8(g, BH * T, D), _i8(g, BH * D, T)
    tp = T + 16  # V^T rows at a pitch: a batch is D rows
    hq, hk = Held(BH * S, D, torch.int8, D + 16, IN_FILL, 0, q), Held(BH * T, D, torch.int8, 2 * D, IN_FILL, 0, k)
    hv, ho = Held(BH * D, T, torch.int8, tp, IN_FILL, 0, vt), Held(BH * S, D, torch.int8, D + 32, OUT_FILL)
    print(f"ti_attention_i8 BH={BH} S={S} T={T} q_len={q_len}", flush=True)
    _ok(L.lib().ti_attention_i8(hq.ptr, S * hq.pitch, hq.pitch, hk.ptr, T * hk.pitch, hk.pitch, hv.ptr, D * tp, tp, ho.ptr, S * ho.pitch,
                                ho.pitch, BH, S, T, D, 1e-3, 0.05, 1.0 / 127, q_len, _stream()), "ti_attention_i8")
    want = fused.attention_i8(q.view(BH, S, D).to(DEV), k.view(BH, T, D).to(DEV), vt.view(BH, D, T).to(DEV), 1e-3, 0.05, 1.0 / 127, q_len)
    assert ho.surroundings_intact() and torch.equal(ho.view.view(BH, S, D), want)


GEMM_CASES = [  # M, N, K, batch, out dtype, epilogue key
    (1, 5, 16, 1, torch.int8), (16, 300, 5120, 1, torch.int8), (5, 40, 48, 2, torch.float32), (129, 257, 1040, 1, torch.int32),
    (300, 1000, 128, 3, torch.int8), (2048, 130, 4096, 1, torch.float32), (70, 6848, 10240, 1, torch.float16),
    (513, 513, 513 * 16, 1, torch.int8), (33, 17, 64, 4, torch.bfloat16), (256, 4096, 4096, 1, torch.int8),
]


@pytest.mark.parametrize("M,N,K,batch,odt", GEMM_CASES)
def test_gemm_stays_inside_its_views(M, N, K, batch, odt):
    """A, B rows at a pitch with NaN-free poison (-1) between them, C rows at a pitch inside a patterned buffer; the
    result equals the same product on contiguous operands."""
    L = _lib()
    g = rng(M * 59 + N + K)
    a, b = _i8(g, batch * M, K), _i8(g, batch * N, K)
    ha, hb = Held(batch * M, K, torch.int8, K + 16, IN_FILL, 0, a), Held(batch * N, K, torch.int8, K + 48, IN_FILL, 0, b)
    hc = Held(batch * M, N, odt, N + 5, OUT_FILL)
    hw = Held(batch * M, N, odt, N, OUT_FILL)
    alpha = torch.tensor([3e-4], device=DEV)
    if odt == torch.int32:
        epi, al = L.EPI_I32, None
    elif odt == torch.int8:
        epi, al = L.EPI_SCALE_I8, alpha.data_ptr()
    else:
        epi, al = L.EPI_SCALE_F, alpha.data_ptr()
    od = L.TORCH_TO_DT[odt]

    def call(A, lda, B, ldb, C, ldc):
        print(f"ti_bmm_i8 M={M} N={N} K={K} batch={batch} {odt} lda={lda} ldb={ldb} ldc={ldc}", flush=True)
        _ok(L.lib().ti_bmm_i8(A, M * lda, lda, 1, B, N * ldb, ldb, 1, C, M * ldc, ldc, 1, batch, M, N, K, None, L.BIAS_NONE, al, None,
                              epi, od, L.ROUND_RNE_CLAMP, _stream()), "ti_bmm_i8")

    call(ha.ptr, ha.pitch, hb.ptr, hb.pitch, hc.ptr, hc.pitch)
    ca, cb = a.to(DEV), b.to(DEV)
    call(ca.data_ptr(), K, cb.data_ptr(), K, hw.ptr, N)
    assert hc.surroundings_intact() and hw.surroundings_intact()
    assert torch.equal(hc.view, hw.view)
    acc = torch.bmm(a.view(batch, M, K).double(), b.view(batch, N, K).double().transpose(1, 2)) if M * N * K * batch < 2e9 else None
    if acc is not None and odt == torch.int32:
        assert torch.equal(hc.view.view(batch, M, N).cpu().double(), acc)


@pytest.mark.parametrize("M,N,K", [(2048, 5120, 512), (1000, 4100, 256), (16, 5120, 2048), (300, 320, 256), (2049, 640, 128)])
def test_linear_with_residual_stays_inside_its_views(M, N, K):
    """ti_linear_i8_residual_f32 with the residual and the output at a pitch inside patterned / poisoned buffers
    (the persistent kernels fetch the residual in their epilogue): equal to the same call on contiguous
    operands, nothing written outside the output's rows."""
    L = _lib()
    g = rng(M * 61 + N + K)
    a, w = _i8(g, M, K), _i8(g, N, K)
    bias, res = _f32(g, 1, N), _f32(g, M, N) * 3
    ha, hw = Held(M, K, torch.int8, K + 16, IN_FILL, 0, a), Held(N, K, torch.int8, K + 32, IN_FILL, 0, w)
    hb, hr = Held(1, N, torch.float32, None, IN_FILL, 0, bias), Held(M, N, torch.float32, N + 12, IN_FILL, 0, res)
    hc, hw2 = Held(M, N, torch.float32, N + 4, OUT_FILL), Held(M, N, torch.float32, N, OUT_FILL)
    alpha, beta = torch.tensor([3e-4], device=DEV), torch.tensor([1.0], device=DEV)
    print(f"ti_linear_i8_residual_f32 M={M} N={N} K={K} pitched", flush=True)
    _ok(L.lib().ti_linear_i8_residual_f32(ha.ptr, ha.pitch, hw.ptr, hw.pitch, hb.ptr, alpha.data_ptr(), beta.data_ptr(), hr.ptr, hr.pitch,
                                          hc.ptr, hc.pitch, M, N, K, _stream()), "ti_linear_i8_residual_f32")
    ca, cw, cb, cr = a.to(DEV), w.to(DEV), bias.to(DEV), res.to(DEV)
    print(f"ti_linear_i8_residual_f32 M={M} N={N} K={K} contiguous", flush=True)
    _ok(L.lib().ti_linear_i8_residual_f32(ca.data_ptr(), K, cw.data_ptr(), K, cb.data_ptr(), alpha.data_ptr(), beta.data_ptr(), cr.data_ptr(), N,
                                          hw2.ptr, N, M, N, K, _stream()), "ti_linear_i8_residual_f32")
    assert hc.surroundings_intact() and hw2.surroundings_intact()
    assert torch.equal(hc.view, hw2.view) and not torch.isnan(hc.view).any()
    acc = a.double() @ w.double().t()
    want = ((acc.float() * 3e-4) + bias.float()) + res  # the three fp32 steps of the contract
    assert torch.equal(hc.view.cpu(), want)
