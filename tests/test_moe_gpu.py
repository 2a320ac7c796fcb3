"""The mixture-of-experts step on a real MI355X, through the C ABI, against oracle/moe_oracle.py:
routing bit for bit (integers) and to fp32 rounding (weights); the gathered product against the grouped
oracle on the permuted rows; activation and combine to one rounding of the output type; the whole layer at
small, Mixtral and fine-grained sizes."""
import pytest
import torch

from grouped_mm_bf16_amd import kernels as K_
from grouped_mm_bf16_amd import moe
from oracle import grouped_mm_oracle as oracle
from oracle import moe_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rnd(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def offs_of(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32)


def check_routing(got: moe.Routing, want: moe_oracle.Routing):
    torch.cuda.synchronize()
    assert torch.equal(got.slot_expert.cpu(), want.slot_expert), "chosen experts differ"
    assert torch.equal(got.offs.cpu(), want.offs), "offs differ"
    assert torch.equal(got.row_token.cpu(), want.row_token), "row order differs"
    assert torch.equal(got.token_rows.cpu(), want.token_rows), "slot -> row map differs"
    torch.testing.assert_close(got.slot_weight.cpu(), want.slot_weight, rtol=2e-5, atol=1e-7)


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (7, 8, 2), (64, 8, 8), (1000, 128, 8), (4096, 128, 8), (8192, 8, 2),
                                   (700, 1023, 32), (3, 70, 1), (300000, 3, 1), (32768, 64, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routing_matches_the_oracle(T, E, k, dtype):
    """bf16 logits tie often: the lower expert index must win, as in a stable descending sort."""
    gen = torch.Generator().manual_seed(T + E + k)
    logits = torch.randn(T, E, generator=gen).to(dtype)
    for renorm in (True, False):
        got = moe.moe_route(logits.to(DEV), k, renormalize=renorm)
        check_routing(got, moe_oracle.route(logits, k, renorm))


def test_routing_fp16_skewed_padded_and_empty():
    gen = torch.Generator().manual_seed(3)
    # skew: most tokens pick expert 0, several experts stay empty
    logits = torch.randn(2048, 32, generator=gen)
    logits[:, 0] += 4.0
    logits[:, 20:] -= 30.0
    lh = logits.half()
    check_routing(moe.moe_route(lh.to(DEV), 2), moe_oracle.route(lh, 2))
    want = moe_oracle.route(lh, 2)
    assert (want.offs[20:] == want.offs[19]).all()
    # a view with a row stride wider than E
    wide = torch.full((2048, 40), float("inf"), device=DEV, dtype=torch.float16)
    wide[:, :32] = lh.to(DEV)
    check_routing(moe.moe_route(wide[:, :32], 2), want)
    # no tokens: offs is all zero, nothing else is written
    r = moe.moe_route(torch.empty(0, 8, device=DEV), 2)
    torch.cuda.synchronize()
    assert r.offs.tolist() == [0] * 8 and r.slot_expert.numel() == 0


@pytest.mark.parametrize("renorm", [True, False])
def test_routing_with_infinite_logits(renorm):
    """-inf masks an expert (weight exactly 0 if it is still chosen); a +inf logit takes all the weight, several
    share it equally; a fully masked row spreads its weight over its choices (renormalised) or over all experts."""
    gen = torch.Generator().manual_seed(21)
    logits = torch.randn(64, 16, generator=gen)
    logits[:, 5:11] = float("-inf")             # masked experts, never among the top 4 of 10 finite ones
    logits[3, :] = float("-inf")                # every expert masked
    logits[4, :14] = float("-inf")              # two finite logits, top_k = 4: two choices are masked experts
    logits[7, 2] = float("inf")
    logits[9, 1] = logits[9, 12] = float("inf")
    got = moe.moe_route(logits.to(DEV), 4, renormalize=renorm)
    want = moe_oracle.route(logits, 4, renorm)
    check_routing(got, want)
    w = got.slot_weight.cpu().view(64, 4)
    assert torch.isfinite(w).all()
    assert w[7].tolist() == [1.0, 0.0, 0.0, 0.0] and w[9].tolist() == [0.5, 0.5, 0.0, 0.0]
    assert w[4, 2:].tolist() == [0.0, 0.0]
    assert w[3].tolist() == ([0.25] * 4 if renorm else [1.0 / 16] * 4)


def test_routing_rejects_what_it_cannot_do():
    lg = torch.zeros(4, 8, device=DEV)
    with pytest.raises(RuntimeError):
        moe.moe_route(lg, 9)
    with pytest.raises(RuntimeError):
        moe.moe_route(lg, 0)
    with pytest.raises(RuntimeError):
        moe.moe_route(torch.zeros(4, 1024, device=DEV), 2)
    with pytest.raises(RuntimeError):
        moe.moe_route(lg.t(), 2)
    from grouped_mm_bf16_amd import _lib
    lib = _lib.load()
    need = lib.gmm_moe_route_workspace_bytes(5000, 128, 8)
    assert need == 40 * 128 * 4
    r = [torch.empty(40000, device=DEV, dtype=torch.int32) for _ in range(5)]
    rc = lib.gmm_moe_route(torch.zeros(5000, 128, device=DEV).data_ptr(), 128, _lib.DT_F32, 5000, 128, 8, 1,
                           r[0].data_ptr(), r[1].data_ptr(), r[2].view(torch.float32).data_ptr(), r[3].data_ptr(),
                           r[4].data_ptr(), r[0].data_ptr(), need - 4, None)
    assert rc == 4 and b"workspace" in lib.gmm_status_string(rc)


# ------------------------------------------------------------------ gathered product
SIZES = [77, 0, 1, 130, 64, 200, 15, 16, 17, 31, 33, 300]


@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("dtype,K,N,path", [(torch.bfloat16, 136, 264, "mfma"), (torch.float16, 136, 264, "mfma"),
                                            (torch.bfloat16, 4096, 512, "mfma"), (torch.bfloat16, 33, 29, "generic"),
                                            (torch.float32, 40, 24, "generic"), (torch.bfloat16, 136, 264, "generic")])
def test_gathered_product_equals_the_product_of_the_gathered_rows(dtype, K, N, path, b_col):
    gen = torch.Generator().manual_seed(K + N)
    G, M, S = len(SIZES), sum(SIZES), 401
    a = rnd(gen, S, K, dtype=dtype)
    b = rnd(gen, G, K, N, dtype=dtype, scale=0.1)
    idx = torch.randint(0, S, (M + 9,), generator=gen).to(torch.int32)   # repeats; 9 rows past offs[-1]
    idx[5], idx[300] = -1, S                                            # outside the source: rows of zeros
    offs = offs_of(SIZES)
    bd = b.to(DEV)
    if b_col:
        bd = bd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((M + 9, N), float("nan"), device=DEV, dtype=dtype)
    with K_.forced_path(path):
        moe.grouped_mm_gathered(a.to(DEV), idx.to(DEV), bd, offs.to(DEV), out=out)
        torch.cuda.synchronize()
        assert K_.last_path() == path
        # the same kernel on a materialised copy: bit-identical
        az = torch.cat([a, torch.zeros(1, K, dtype=dtype)])
        src = idx.long().clone()
        src[(src < 0) | (src >= S)] = S
        plain = torch.full_like(out, float("nan"))
        K_.grouped_mm_2d3d(az[src].to(DEV), bd, offs.to(DEV), plain)
        torch.cuda.synchronize()
    got = out.cpu()
    assert torch.isnan(got[M:].float()).all(), "rows past offs[-1] were written"
    assert torch.equal(got[:M].view(torch.int16 if dtype != torch.float32 else torch.int32),
                       plain.cpu()[:M].view(torch.int16 if dtype != torch.float32 else torch.int32))
    want = oracle.grouped_mm(az[src], b, offs)
    if dtype == torch.float32:
        torch.testing.assert_close(got[:M], want[:M], rtol=3e-4, atol=3e-4)
    else:
        oracle.assert_close(got[:M], want[:M], K)
    assert (got[5] == 0).all() and (got[300] == 0).all()


def test_gathered_product_on_views_and_large_sources():
    """Source rows 24 elements apart from their extent, at a storage offset; a source whose byte offsets need
    all 31 bits still takes the assembly tile, a larger one goes to the generic family."""
    gen = torch.Generator().manual_seed(77)
    K, N, S = 136, 264, 90
    a = rnd(gen, S, K)
    buf = torch.full((16 + S * (K + 24) - 24,), float("nan"), device=DEV, dtype=torch.bfloat16)
    av = torch.as_strided(buf, (S, K), (K + 24, 1), 16)
    av.copy_(a)
    sizes = [40, 0, 3, 100]
    idx = torch.randint(0, S, (sum(sizes),), generator=gen).to(torch.int32)
    b = rnd(gen, len(sizes), K, N, scale=0.1)
    with K_.forced_path("mfma"):
        got = moe.grouped_mm_gathered(av, idx.to(DEV), b.to(DEV), offs_of(sizes).to(DEV))
        torch.cuda.synchronize()
    oracle.assert_close(got.cpu(), oracle.grouped_mm(a[idx.long()], b, offs_of(sizes)), K)
    # 2^31 bytes of source: rows * ld * 2 == 2^31 exactly is refused by the tile, taken by the generic kernels
    S2, K2 = 1 << 17, 8192
    big = torch.zeros(S2, K2, device=DEV, dtype=torch.bfloat16)
    big[S2 - 1] = 1.0
    idx2 = torch.tensor([S2 - 1, 0, S2 - 1], dtype=torch.int32, device=DEV)
    b2 = torch.ones(1, K2, 8, device=DEV, dtype=torch.bfloat16)
    got = moe.grouped_mm_gathered(big, idx2, b2, torch.tensor([3], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert K_.last_path() == "generic"
    assert got.float().cpu().tolist() == [[8192.0] * 8, [0.0] * 8, [8192.0] * 8]
    got = moe.grouped_mm_gathered(big[: S2 - 8], idx2 - 8, b2, torch.tensor([3], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert K_.last_path() == "mfma"
    assert got.float().cpu().tolist() == [[0.0] * 8, [0.0] * 8, [0.0] * 8]
    idx3 = torch.tensor([S2 - 9, S2 - 1, 0], dtype=torch.int32, device=DEV)   # last valid row; out of range; first
    big[S2 - 9] = 2.0
    got = moe.grouped_mm_gathered(big[: S2 - 8], idx3, b2, torch.tensor([3], dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    assert got.float().cpu().tolist() == [[16384.0] * 8, [0.0] * 8, [0.0] * 8]


# ------------------------------------------------------------------ product with the SwiGLU epilogue
@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("gather", [False, True])
@pytest.mark.parametrize("dtype,K,N", [(torch.bfloat16, 136, 256), (torch.float16, 136, 384), (torch.bfloat16, 2048, 1536)])
def test_fused_swiglu_product(dtype, K, N, gather, b_col):
    """out = swiglu(a[idx] @ b[g]) from the fp32 accumulators, b in the interleaved layout; against the oracle
    (activation of the fp32 product, one rounding) and against the two-kernel path on the same device."""
    gen = torch.Generator().manual_seed(K + N)
    G, M, S = len(SIZES), sum(SIZES), 401
    a = rnd(gen, S if gather else M + 9, K, dtype=dtype)
    w = rnd(gen, G, K, N, dtype=dtype, scale=K ** -0.5)                   # plain layout [gate | up]
    idx = torch.randint(0, S, (M + 9,), generator=gen).to(torch.int32) if gather else None
    offs = offs_of(SIZES)
    wd = moe.interleave_gate_up(w.to(DEV))
    if b_col:
        wd = wd.transpose(1, 2).contiguous().transpose(1, 2)
    out = torch.full((M + 9, N // 2), float("nan"), device=DEV, dtype=dtype)
    moe.grouped_mm_swiglu(a.to(DEV), idx.to(DEV) if gather else None, wd, offs.to(DEV), out=out)
    torch.cuda.synchronize()
    assert K_.last_path() == "mfma"
    got = out.cpu()
    assert torch.isnan(got[M:].float()).all(), "rows past offs[-1] were written"
    rows = a[idx.long()] if gather else a
    h32 = oracle.grouped_mm(rows, w, offs, out_dtype=torch.float32)
    want = moe_oracle.activation(h32[:M], "swiglu").to(dtype)
    # |d swiglu| <= ~1.1 |dg| |u| + |du|: the product's bar carries over with the size of the partner
    oracle.assert_close(got[:M], want, K)
    ulp_like = (got[:M].float() - want.float()).abs() <= 2.0 ** -6 * want.float().abs() + 2e-3
    assert ulp_like.float().mean() > 0.999
    # two kernels: product rounded to 16 bits, then the activation kernel
    h16 = torch.empty(M + 9, N, device=DEV, dtype=dtype)
    if gather:
        moe.grouped_mm_gathered(a.to(DEV), idx.to(DEV), w.to(DEV), offs.to(DEV), out=h16)
    else:
        K_.grouped_mm_2d3d(a.to(DEV), w.to(DEV), offs.to(DEV), h16)
    two = moe.moe_activation(h16[:M], "swiglu").cpu()
    oracle.assert_close(got[:M], two, K)


def test_fused_swiglu_rejects_what_the_tile_cannot_do():
    a = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    offs = torch.tensor([64], device=DEV, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="unsupported"):
        moe.grouped_mm_swiglu(a, None, torch.zeros(1, 64, 192, device=DEV, dtype=torch.bfloat16), offs)   # N % 128
    with pytest.raises(RuntimeError, match="unsupported"):
        moe.grouped_mm_swiglu(a.float(), None, torch.zeros(1, 64, 256, device=DEV), offs)                  # fp32
    with pytest.raises(RuntimeError, match="unsupported"):
        moe.grouped_mm_swiglu(a.t().contiguous().t(), None, torch.zeros(1, 64, 256, device=DEV, dtype=torch.bfloat16), offs)
    with K_.forced_path("generic"), pytest.raises(RuntimeError, match="unsupported"):
        moe.grouped_mm_swiglu(a, None, torch.zeros(1, 64, 256, device=DEV, dtype=torch.bfloat16), offs)


# ------------------------------------------------------------------ activation, combine
def ulp_close(got, want, dtype):
    """Equal up to one unit in the last place of the 16-bit type (fast exp and fused multiply-adds on the device)."""
    eps = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    torch.testing.assert_close(got.float(), want.float(), rtol=eps, atol=1e-6 if dtype == torch.bfloat16 else 1e-7)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["silu", "swiglu"])
def test_activation(kind, dtype):
    gen = torch.Generator().manual_seed(21)
    h = rnd(gen, 333, 272, dtype=dtype, scale=3.0)
    h[0, :8] = torch.tensor([0.0, -0.0, 80.0, -80.0, float("inf"), 1e-3, -1e-3, 11.0]).to(dtype)
    got = moe.moe_activation(h.to(DEV), kind).cpu()
    want = moe_oracle.activation(h, kind)
    assert got.shape == want.shape
    ok = torch.isfinite(want.float())
    ulp_close(got[ok], want[ok], dtype)
    # a view: rows of a wider matrix
    wide = torch.full((333, 304), float("nan"), device=DEV, dtype=dtype)
    wide[:, :272] = h.to(DEV)
    got2 = moe.moe_activation(wide[:, :272], kind).cpu()
    assert torch.equal(got2.view(torch.int16), got.view(torch.int16))
    assert moe.moe_activation(torch.empty(0, 16, device=DEV, dtype=dtype), kind).shape == (0, 8 if kind == "swiglu" else 16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,k,H", [(1, 1, 8), (50, 2, 264), (300, 8, 2048), (17, 32, 40)])
def test_combine(T, k, H, dtype):
    gen = torch.Generator().manual_seed(T + k + H)
    E = 40
    r = moe_oracle.route(torch.randn(T, E, generator=gen), k)
    y = rnd(gen, T * k, H, dtype=dtype)
    dev_r = moe.Routing(*(t.to(DEV) for t in r))
    got = moe.moe_combine(y.to(DEV), dev_r, T, k).cpu()
    ulp_close(got, moe_oracle.combine(y, r, T, k), dtype)
    # a slot that points outside y adds nothing
    rows = r.token_rows.clone()
    rows[0] = T * k
    rows[-1] = -1
    r2 = r._replace(token_rows=rows)
    got = moe.moe_combine(y.to(DEV), moe.Routing(*(t.to(DEV) for t in r2)), T, k).cpu()
    y0 = torch.cat([y, torch.zeros(1, H, dtype=dtype)])
    rows0 = rows.clone()
    rows0[rows0 < 0] = T * k
    ulp_close(got, moe_oracle.combine(y0, r2._replace(token_rows=rows0), T, k), dtype)


# ------------------------------------------------------------------ the whole layer
def layer_case(seed, T, H, I, E, k, kind, dtype=torch.bfloat16, skew=0.0, wscale=None, on_device=False):
    """Inputs with unit-size activations at every stage; big cases draw x and the weights on the device (the
    host generator needs most of a minute for Mixtral's two billion weights) and copy them back for the oracle."""
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=gen)
    if skew:
        logits += skew * torch.randn(E, generator=gen)
    n_up = 2 * I if kind == "swiglu" else I
    s_up, s_down = (wscale, wscale) if wscale else (H ** -0.5, 2 * I ** -0.5)
    if on_device:
        dgen = torch.Generator(device=DEV).manual_seed(seed)
        mk = lambda *shape, scale: (torch.randn(*shape, generator=dgen, device=DEV) * scale).to(dtype).cpu()
        return mk(T, H, scale=1.0), logits, mk(E, H, n_up, scale=s_up), mk(E, I, H, scale=s_down)
    return (rnd(gen, T, H, dtype=dtype), logits, rnd(gen, E, H, n_up, dtype=dtype, scale=s_up),
            rnd(gen, E, I, H, dtype=dtype, scale=s_down))


def run_layer(x, logits, w_up, w_down, k, kind, renorm=True, fused=False):
    wu = moe.interleave_gate_up(w_up.to(DEV)) if fused else w_up.to(DEV)
    got = moe.moe_forward(x.to(DEV), logits.to(DEV), wu, w_down.to(DEV), k, kind, renorm, interleaved=fused)
    torch.cuda.synchronize()
    want = moe_oracle.moe_forward(x, logits, w_up, w_down, k, kind, renorm, fused=fused)
    # three stages, each within the grouped product's bar; the last contraction runs over I
    oracle.assert_close(got.cpu(), want, w_down.shape[1])
    # and as a whole far inside one rounding of the 16-bit type (differences come from rounding flips only)
    rel = float((got.cpu().double() - want.double()).norm() / want.double().norm())
    assert rel < 4e-3, rel
    return got


@pytest.mark.parametrize("kind", ["silu", "swiglu"])
@pytest.mark.parametrize("T,H,I,E,k", [(1, 64, 64, 4, 1), (130, 136, 264, 6, 2), (257, 256, 512, 16, 4), (64, 128, 72, 128, 8)])
def test_layer_small(T, H, I, E, k, kind):
    case = layer_case(T + E, T, H, I, E, k, kind)
    run_layer(*case, k, kind)
    run_layer(*case, k, kind, renorm=False)


@pytest.mark.parametrize("T,H,I,E,k", [(130, 136, 256, 6, 2), (257, 256, 512, 16, 4), (64, 128, 64, 128, 8)])
def test_layer_small_fused(T, H, I, E, k):
    run_layer(*layer_case(T + E, T, H, I, E, k, "swiglu"), k, "swiglu", fused=True)


def test_layer_fp16_and_dense_pin():
    """fp16; and the device result against the token-by-token fp64 formulation directly."""
    x, logits, w_up, w_down = layer_case(5, 48, 64, 96, 5, 2, "swiglu", dtype=torch.float16)
    got = run_layer(x, logits, w_up, w_down, 2, "swiglu")
    dense = moe_oracle.moe_dense(x, logits, w_up, w_down, 2, "swiglu")
    torch.testing.assert_close(got.cpu().double(), dense, rtol=2e-2, atol=2e-3)


def test_layer_mixtral_size():
    """8192 tokens, hidden 4096, inner 14336, 8 experts, top 2, SwiGLU: the up projection is the headline
    workload with the gate and up weights side by side."""
    x, logits, w_up, w_down = layer_case(0, 8192, 4096, 14336, 8, 2, "swiglu", wscale=0.02, on_device=True)
    logits[:, 0] += 1.0
    run_layer(x, logits, w_up, w_down, 2, "swiglu")
    assert K_.last_path() == "mfma"
    run_layer(x, logits, w_up, w_down, 2, "swiglu", fused=True)


def test_layer_fine_grained_size():
    """4096 tokens, hidden 2048, inner 768, 128 experts, top 8, skewed popularity (empty and one-row experts)."""
    x, logits, w_up, w_down = layer_case(1, 4096, 2048, 768, 128, 8, "swiglu", skew=1.5, wscale=0.02, on_device=True)
    r = moe_oracle.route(logits, 8)
    sizes = torch.diff(r.offs, prepend=torch.zeros(1, dtype=torch.int32))
    assert (sizes == 0).sum() > 10 and (sizes == 1).any() and (sizes < 16).sum() > 40
    run_layer(x, logits, w_up, w_down, 8, "swiglu")
    assert K_.last_path() == "mfma"
    run_layer(x, logits, w_up, w_down, 8, "swiglu", fused=True)


def test_layer_replays_from_a_captured_graph():
    """The whole layer on static buffers -- routing through the entry point that allocates nothing, fused up
    projection, down projection, combine -- captured once and replayed on new tokens and new router logits: the
    routing, and with it `offs`, changes from replay to replay without the host ever seeing it.  Every replay
    must equal the eager layer on the same inputs bit for bit, and the oracle within the bar."""
    from grouped_mm_bf16_amd import _lib
    lib = _lib.load()
    T, H, I, E, k = 300, 256, 256, 16, 4
    S = T * k
    gen = torch.Generator().manual_seed(99)
    w_up, w_down = rnd(gen, E, H, 2 * I, scale=H ** -0.5), rnd(gen, E, I, H, scale=2 * I ** -0.5)
    w_il, w_dn = moe.interleave_gate_up(w_up.to(DEV)), w_down.to(DEV)
    x_s = torch.zeros(T, H, device=DEV, dtype=torch.bfloat16)
    lg_s = torch.zeros(T, E, device=DEV)
    i32 = dict(device=DEV, dtype=torch.int32)
    r = moe.Routing(torch.zeros(E, **i32), torch.zeros(S, **i32), torch.zeros(S, device=DEV), torch.zeros(S, **i32),
                    torch.zeros(S, **i32))
    act = torch.zeros(S, I, device=DEV, dtype=torch.bfloat16)
    y = torch.zeros(S, H, device=DEV, dtype=torch.bfloat16)
    out_s = torch.zeros(T, H, device=DEV, dtype=torch.bfloat16)

    def layer():
        rc = lib.gmm_moe_route_noalloc(lg_s.data_ptr(), E, _lib.DT_F32, T, E, k, 1, r.offs.data_ptr(), r.slot_expert.data_ptr(),
                                       r.slot_weight.data_ptr(), r.row_token.data_ptr(), r.token_rows.data_ptr(),
                                       torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        moe.grouped_mm_swiglu(x_s, r.row_token, w_il, r.offs, out=act)
        K_.grouped_mm_2d3d(act, w_dn, r.offs, y)
        moe.moe_combine(y, r, T, k, out=out_s)

    layer()                                       # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            layer()
    torch.cuda.current_stream().wait_stream(side)
    seen = set()
    for rep in range(3):
        x, logits = rnd(gen, T, H), torch.randn(T, E, generator=gen) + rep * torch.randn(E, generator=gen)
        x_s.copy_(x.to(DEV))
        lg_s.copy_(logits.to(DEV))
        out_s.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        replayed = out_s.clone()
        seen.add(tuple(r.offs.tolist()))
        eager = moe.moe_forward(x_s, lg_s, w_il, w_dn, k, interleaved=True)
        torch.cuda.synchronize()
        assert torch.equal(replayed.view(torch.int16), eager.view(torch.int16)), f"replay {rep} differs from eager"
        oracle.assert_close(replayed.cpu(), moe_oracle.moe_forward(x, logits, w_up, w_down, k, fused=True), I)
    assert len(seen) == 3, "the routing was meant to change between replays"


# ------------------------------------------------------------------ the step as torch custom ops
@pytest.mark.parametrize("fused", [False, True])
def test_compiled_layer_goes_through_the_custom_ops(fused):
    """torch.compile(fullgraph=True) of a function that calls moe_forward: every stage is reached through its
    registered op (no graph break), and the compiled layer returns what the eager layer returns, bit for bit."""
    T, H, I, E, k = 130, 136, 256, 6, 2
    x, logits, w_up, w_down = layer_case(77, T, H, I, E, k, "swiglu")
    wu = moe.interleave_gate_up(w_up.to(DEV)) if fused else w_up.to(DEV)
    args = (x.to(DEV), logits.to(DEV), wu, w_down.to(DEV))

    def layer(x_, lg_, wu_, wd_):
        return moe.moe_forward(x_, lg_, wu_, wd_, k, "swiglu", True, interleaved=fused) * 2.0

    eager = layer(*args)
    torch._dynamo.reset()
    compiled = torch.compile(layer, backend="aot_eager", fullgraph=True)(*args)
    torch.cuda.synchronize()
    assert torch.equal(eager.view(torch.int16), compiled.view(torch.int16))
    want = moe_oracle.moe_forward(x, logits, w_up, w_down, k, "swiglu", True, fused=fused) * 2.0
    oracle.assert_close(compiled.cpu(), want, I)


def test_custom_ops_pass_opcheck_and_match_the_direct_calls():
    T, H, I, E, k = 70, 136, 128, 5, 2
    x, logits, w_up, w_down = layer_case(78, T, H, I, E, k, "swiglu")
    xd, lg, wu = x.to(DEV), logits.to(DEV), w_up.to(DEV)
    ops, checks = torch.ops.grouped_mm_bf16_amd, ("test_schema", "test_faketensor")
    r = moe.moe_route(lg, k)
    packed = ops.moe_route(lg, k, True)
    assert torch.equal(packed[:E], r.offs) and torch.equal(packed[E + 2 * T * k:E + 3 * T * k], r.row_token)
    torch.library.opcheck(ops.moe_route.default, (lg, k, True), test_utils=checks)
    h = moe.grouped_mm_gathered(xd, r.row_token, wu, r.offs)
    assert torch.equal(ops.gathered(xd, r.row_token, wu, r.offs).view(torch.int16), h.view(torch.int16))
    torch.library.opcheck(ops.gathered.default, (xd, r.row_token, wu, r.offs), test_utils=checks)
    wil = moe.interleave_gate_up(wu)
    fused = moe.grouped_mm_swiglu(xd, r.row_token, wil, r.offs)
    assert torch.equal(ops.swiglu(xd, r.row_token, wil, r.offs).view(torch.int16), fused.view(torch.int16))
    torch.library.opcheck(ops.swiglu.default, (xd, r.row_token, wil, r.offs), test_utils=checks)
    torch.library.opcheck(ops.swiglu.default, (fused, None, wil[:, :I], r.offs), test_utils=checks)
    act = moe.moe_activation(h, "swiglu")
    assert torch.equal(ops.activation(h, "swiglu").view(torch.int16), act.view(torch.int16))
    torch.library.opcheck(ops.activation.default, (h, "silu"), test_utils=checks)
    y = torch.empty(T * k, H, device=DEV, dtype=torch.bfloat16)
    K_.grouped_mm_2d3d(act, w_down.to(DEV), r.offs, y)
    out = moe.moe_combine(y, r, T, k)
    assert torch.equal(ops.combine(y, r.token_rows, r.slot_weight, T, k).view(torch.int16), out.view(torch.int16))
    torch.library.opcheck(ops.combine.default, (y, r.token_rows, r.slot_weight, T, k), test_utils=checks)
