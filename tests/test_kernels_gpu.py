"""Each HIP kernel alone against a plain PyTorch float32 computation of the same op, at
sizes other than the engine tests' (head sizes in steps of 16, widths and vocabularies
that are no power of two, odd row counts)."""
import math

import pytest
import torch

from util import from_cache_order, to_cache_order

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def K():
    from gpt_fast_amd.ops import kernels
    return kernels


def bf(t):
    return t.to(torch.bfloat16)


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err < tol, err


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    torch.manual_seed(0)
    table = torch.randn(333, 72, device=DEV).to(dtype)
    tok = torch.tensor([0, 332, 5, 5, 17], dtype=torch.int32, device=DEV)
    assert torch.equal(K().embed(table, tok), table[tok.long()].float())


@pytest.mark.parametrize("dim,eps", [(72, 1e-5), (200, 1e-6), (4096, 1e-5), (1000, 0.3)])
def test_rmsnorm(dim, eps):
    torch.manual_seed(1)
    x = torch.randn(7, dim, device=DEV) * 3
    w = torch.randn(dim, device=DEV)
    ref = x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()
    close(K().rmsnorm(x, w, eps, torch.float32), ref, 2e-6)
    close(K().rmsnorm(x, w, eps, torch.bfloat16), ref, 1e-2)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(K().rmsnorm(x, w, eps, torch.float32, rows=rows),
                       K().rmsnorm(x, w, eps, torch.float32)[rows.long()])
    # eps inside the root: it dominates a tiny input
    tiny = torch.full((1, dim), 1e-4, device=DEV)
    out = K().rmsnorm(tiny, torch.ones(dim, device=DEV), 1e-2, torch.float32)
    close(out, tiny / math.sqrt(1e-8 + 1e-2), 1e-5)


@pytest.mark.parametrize("rows,dim,eps", [(3, 72, 1e-5), (40, 200, 1e-6), (17, 4096, 1e-5),
                                          (5, 6144, 1e-5), (9, 1001, 0.3)])
def test_residual_sum_and_rmsnorm_in_one_pass(rows, dim, eps):
    torch.manual_seed(12)
    res0 = torch.randn(rows, dim, device=DEV) * 3
    res0[0] *= 40.0
    y = bf(torch.randn(rows, dim, device=DEV))
    g = 1 + 0.1 * torch.randn(dim, device=DEV)
    res = res0.clone()
    out = K().add_rmsnorm(res, y, g, eps)
    want_res = res0 + y.float()
    assert torch.equal(res, want_res)
    r = want_res.double()
    close(out, r * torch.rsqrt((r ** 2).mean(-1, keepdim=True) + eps) * g.double(), 6e-3)
    # the two separate kernels give the same rows
    sep = res0.clone()
    K().add_into(sep, y)
    close(out, K().rmsnorm(sep, g, eps, torch.bfloat16), 6e-3)


@pytest.mark.parametrize("M,N,K_", [(1, 5, 3), (3, 100, 70), (65, 130, 257), (200, 64, 1000)])
def test_gemm_f32(M, N, K_):
    torch.manual_seed(2)
    a = torch.randn(M, K_, device=DEV)
    w = torch.randn(N, K_, device=DEV)
    ref = a.double() @ w.double().T
    out = K().gemm_f32(a, w)
    close(out, ref, 1e-5)
    # rows do not depend on the other rows: a float32 result is the same for any cutting
    assert torch.equal(K().gemm_f32(a[M // 2:M // 2 + 1], w), out[M // 2:M // 2 + 1])
    res = torch.randn(M, N, device=DEV)
    keep = res.clone()
    K().gemm_f32(a, w, out=res, accumulate=True)
    close(res, keep.double() + ref, 1e-5)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 9, 16, 17, 20, 22, 24, 33, 64])
@pytest.mark.parametrize("N,K_", [(40, 64), (136, 200), (1000, 328), (96, 4096), (77, 75)])
def test_skinny_bf16(M, N, K_):
    from gpt_fast_amd.ops import gemm_bf16 as G
    torch.manual_seed(3)
    x = bf(torch.randn(M, K_, device=DEV))
    w = bf(torch.randn(N, K_, device=DEV) * 0.1)
    ref = x.double() @ w.double().T
    close(G.skinny(x, w, out_dtype=torch.float32), ref, 2e-5)
    close(G.skinny(x, w, out_dtype=torch.bfloat16), ref, 1e-2)
    res = torch.randn(M, N, device=DEV)
    keep = res.clone()
    G.skinny(x, w, residual=res)
    close(res, keep.double() + ref, 2e-5)
    close(K().gemm_bf16_naive(x, w), ref, 2e-5)
    if N % 2 == 0:
        I = N // 2
        g = ref[:, :I]
        close(G.skinny_gated(x, w), (g * torch.sigmoid(g)) * ref[:, I:], 1.5e-2)


@pytest.mark.parametrize("M", [3, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K_", [(40, 64), (136, 200), (1000, 328), (256, 4096), (77, 72), (4096, 1024)])
def test_products_of_up_to_64_rows(M, N, K_):
    """The kernels for 17..64 rows (shared x in LDS, K in slices): plain, float, into the
    residual stream with and without the norm that follows, and gated."""
    from gpt_fast_amd.ops import gemm_wide_bf16 as W
    torch.manual_seed(14)
    x = bf(torch.randn(M, K_, device=DEV))
    w = bf(torch.randn(N, K_, device=DEV) * 0.1)
    ref = x.double() @ w.double().T
    close(W.product(x, w, torch.float32), ref, 2e-5)
    close(W.product(x, w), ref, 6e-3)
    res0 = torch.randn(M, N, device=DEV)
    res = res0.clone()
    assert W.product_into(x, w, res) is None
    close(res, res0.double() + ref, 2e-5)
    if N % 4 == 0:
        g = 1 + 0.1 * torch.randn(N, device=DEV)
        res2 = res0.clone()
        xn = W.product_into(x, w, res2, g, 1e-5)
        close(res2, res0.double() + ref, 2e-5)
        if xn is not None:                                 # sliced: the norm rode along
            assert W.slices(M, N, K_) > 1
            r = res2.double()
            close(xn, r * torch.rsqrt((r ** 2).mean(-1, keepdim=True) + 1e-5) * g.double(), 6e-3)
    if N % 2 == 0:
        I = N // 2
        a = ref[:, :I]
        close(W.product_gated(x, w), (a * torch.sigmoid(a)) * ref[:, I:], 1e-2)


def _tiled_by_hand(w, gate):
    """The tiled form written from its description: [tiles][Kp / 8][16][8], Kp = K rounded up to
    128, zeros beyond the matrix; gate: tile t = rows 8 t .. + 7 of W1, then the same rows of W3."""
    rows, K = w.shape
    Kp = (K + 127) // 128 * 128
    if gate:
        I = rows // 2
        tiles = (I + 7) // 8
        src = torch.zeros(tiles, 16, Kp, dtype=w.dtype)
        for t in range(tiles):
            n = min(8, I - 8 * t)
            src[t, :n, :K] = w[8 * t:8 * t + n]
            src[t, 8:8 + n, :K] = w[I + 8 * t:I + 8 * t + n]
    else:
        tiles = (rows + 15) // 16
        src = torch.zeros(tiles * 16, Kp, dtype=w.dtype)
        src[:rows, :K] = w
        src = src.view(tiles, 16, Kp)
    return src.view(tiles, 16, Kp // 8, 8).permute(0, 2, 1, 3).contiguous().view(-1)


@pytest.mark.parametrize("M", [17, 25, 32, 33, 48, 64, 3])
@pytest.mark.parametrize("N,K_", [(40, 64), (136, 200), (1000, 328), (256, 4096), (77, 72), (4096, 1024),
                                  (6144, 512), (2000, 1536)])
def test_products_over_weights_in_operand_order(M, N, K_):
    """The 17..64-row kernels that read W in the matrix cores' operand order: the tiled copy
    itself, the partial sums of a sliced product (added in slice order), the one-kernel float
    product, and the gate with its eight-and-eight tiles - at widths and inner sizes that are
    no multiples of the tile (16 rows of W, 128 values of k), against float64."""
    from gpt_fast_amd.ops import gemm_tiled_bf16 as T
    torch.manual_seed(M + N)
    x = bf(torch.randn(M, K_))
    w = bf(torch.randn(N, K_) / math.sqrt(K_))
    ref = x.double() @ w.double().T
    t = T.tile(w.to(DEV))
    assert torch.equal(t.data.cpu(), _tiled_by_hand(w, False))
    part = T.partial_sums(x.to(DEV), t)
    assert part.shape[1:] == (M, N) and part.shape[0] == T.slices(N, K_)
    close(part.sum(0), ref, 1e-5)
    close(T.product_f32(x.to(DEV), t), ref, 1e-5)
    if N % 2 == 0:
        I = N // 2
        tg = T.tile(w.to(DEV), gate=True)
        assert torch.equal(tg.data.cpu(), _tiled_by_hand(w, True))
        a, b = ref[:, :I], ref[:, I:]
        close(T.product_gated(x.to(DEV), tg), a * torch.sigmoid(a) * b, 1.5e-2)


@pytest.mark.parametrize("M,N,K_", [(300, 512, 4096), (129, 256, 8192), (700, 1024, 2048)])
def test_many_row_products_in_slices_of_the_inner_size(M, N, K_):
    """More than 64 rows times a matrix with few tiles: the vendor library's batched product
    over slices of the inner size (float32 partial sums), added by the kernel that completes
    the residual stream and norms it, or kept for a reader that adds them; against float64."""
    from gpt_fast_amd.ops import linear as L
    torch.manual_seed(M)
    S = L._library_slices(M, N, K_, torch.device(DEV))
    assert S > 1 and K_ % S == 0
    x = bf(torch.randn(M, K_, device=DEV))
    w = bf(torch.randn(N, K_, device=DEV) / math.sqrt(K_))
    ref = x.double() @ w.double().T
    part = L._library_partial_sums(x, w, S)
    assert part.shape == (S, M, N) and part.dtype == torch.float32 and part.is_contiguous()
    per = K_ // S
    for i in (0, S - 1):
        close(part[i], x[:, i * per:(i + 1) * per].double() @ w[:, i * per:(i + 1) * per].double().T, 2e-5)
    res0 = torch.randn(M, N, device=DEV)
    g, eps = (1 + 0.1 * torch.randn(N, device=DEV)).float(), 1e-5

    class Norm:
        def row_and_column_form(self):
            return g, eps

    res = res0.clone()
    xn = L.linear_into(x, w, res, Norm())
    r = res0.double() + ref
    close(res, r, 2e-5)
    close(xn, r * torch.rsqrt((r ** 2).mean(-1, keepdim=True) + eps) * g.double(), 6e-3)
    res = res0.clone()
    assert L.linear_into(x, w, res) is None
    close(res, r, 2e-5)
    rows = L.linear(x, w, may_stay_sliced=True)
    assert isinstance(rows, L.SlicedRows) and rows.part.shape[0] == S
    close(rows.rows(), ref, 1e-2)
    close(L.linear(x, w), ref, 1e-2)


def test_products_of_17_to_64_rows_without_room_for_the_second_copy(monkeypatch):
    """The tiled copy of a weight matrix is only made while enough of the device's memory
    stays free; a matrix that was refused one is asked for no other, and its products run on
    the kernels over the row-major matrix with the same results."""
    from gpt_fast_amd.ops import gemm_tiled_bf16 as T
    from gpt_fast_amd.ops import linear as L
    torch.manual_seed(3)
    M, N, K_ = 40, 512, 1024
    x = bf(torch.randn(M, K_, device=DEV))
    w = bf(torch.randn(N, K_, device=DEV) / math.sqrt(K_))
    w13 = bf(torch.randn(2 * N, K_, device=DEV) / math.sqrt(K_))
    ref = x.double() @ w.double().T
    a = x.double() @ w13.double().T
    gated = a[:, :N] * torch.sigmoid(a[:, :N]) * a[:, N:]
    res0 = torch.randn(M, N, device=DEV)
    with monkeypatch.context() as m:
        m.setattr(T, "KEEP_FREE_FRACTION", 2.0)            # never enough room
        assert T.tiled_of(w) is None and w._gfa_tiled_refused
        assert T.tiled_of(w13, gate=True) is None
        close(L.linear(x, w), ref, 1e-2)
        close(L.gated_linear(x, w13), gated, 1.5e-2)
        res = res0.clone()
        L.linear_into(x, w, res)
        close(res, res0.double() + ref, 2e-5 if L._sliced_is_faster(M, N, K_) else 1e-2)
    assert T.tiled_of(w) is None                           # asked once: the refusal stands
    w_again = w.clone()
    assert T.tiled_of(w_again) is not None                 # room now: another tensor gets its copy
    close(L.linear(x, w_again), ref, 1e-2)
    res = res0.clone()
    L.linear_into(x, w_again, res)
    close(res, res0.double() + ref, 2e-5)


def test_sliced_product_equals_its_slices_added_in_order():
    from gpt_fast_amd.ops import gemm_wide_bf16 as W
    torch.manual_seed(15)
    M, N, K_ = 40, 512, 4096
    x = bf(torch.randn(M, K_, device=DEV))
    w = bf(torch.randn(N, K_, device=DEV) * 0.1)
    part = W.partial_sums(x, w)
    S = part.shape[0]
    assert S == W.slices(M, N, K_) and S > 1
    total = part[0].clone()
    for s in range(1, S):
        total += part[s]
    assert torch.equal(W.sum_store(part, torch.float32), total)
    per = ((K_ + 127) // 128 + S - 1) // S * 128
    for s in (0, S - 1):
        close(part[s], x[:, s * per:(s + 1) * per].double() @ w[:, s * per:(s + 1) * per].double().T, 2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul_and_add_into(dtype):
    torch.manual_seed(4)
    gu = torch.randn(5, 2 * 37, device=DEV).to(dtype)
    ref = torch.nn.functional.silu(gu[:, :37].double()) * gu[:, 37:].double()
    close(K().silu_mul(gu), ref, 1e-6 if dtype == torch.float32 else 1e-2)
    res = torch.randn(5, 37, device=DEV)
    y = torch.randn(5, 37, device=DEV).to(dtype)
    want = res + y.float()
    assert torch.equal(K().add_into(res, y), want)


def _paged(S_list, G, hd, dtype, seed):
    """Random keys/values for sequences of the given lengths scattered over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum((s + 63) // 64 for s in S_list) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    k_pages = torch.full((n_pages, G, 64, hd), float("nan")).to(dtype)      # poison: never read
    v_pages = torch.full((n_pages, G, hd, 64), float("nan")).to(dtype)     # values transposed
    width = max((s + 63) // 64 for s in S_list)
    table = torch.full((len(S_list), width), -1, dtype=torch.int32)
    ks, vs = [], []
    for b, S in enumerate(S_list):
        k = torch.randn(S, G, hd, generator=g).to(dtype)
        v = torch.randn(S, G, hd, generator=g).to(dtype)
        ks.append(k)
        vs.append(v)
        for i in range((S + 63) // 64):
            p = perm.pop()
            table[b, i] = p
            n = min(64, S - 64 * i)
            k_pages[p, :, :n] = k[64 * i:64 * i + n].transpose(0, 1)
            v_pages[p, :, :, :n] = v[64 * i:64 * i + n].permute(1, 2, 0)
    k_pages, v_pages = to_cache_order(k_pages, v_pages)
    return k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), ks, vs


def _attention_ref(q, k, v, pos, scale, window):
    """q [H, hd] at position pos over k, v [S, G, hd] in float64."""
    H, hd = q.shape
    G = k.shape[1]
    lo = max(0, pos - window + 1) if window else 0
    out = torch.empty(H, hd, dtype=torch.float64)
    for h in range(H):
        g = h // (H // G)
        s = (k[lo:pos + 1, g].double() @ q[h].double()) * scale
        out[h] = torch.softmax(s, 0) @ v[lo:pos + 1, g].double()
    return out


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("H,G,hd,window", [
    (4, 4, 16, 0), (6, 2, 48, 0), (8, 1, 128, 0), (3, 3, 80, 0), (4, 2, 64, 37), (2, 1, 256, 100),
    (32, 1, 64, 0),                 # 32 heads on one kv head: two row tiles per token
    (7, 7, 32, 0), (10, 2, 112, 0), (9, 3, 96, 65), (5, 1, 144, 0), (2, 2, 176, 0), (3, 1, 208, 0),
    (2, 1, 240, 0), (12, 4, 128, 33), (4, 1, 20, 0), (2, 2, 264, 0),      # last two: plain kernel only
])
def test_attention_over_pages(dtype, tol, H, G, hd, window, monkeypatch):
    """Prefill rows (many tokens of a sequence) and decode rows (its last token) in one
    launch, sequences of unequal length on scattered pages, unused page tails poisoned.
    The workgroup-tiled prompt kernel is run in both its tile heights (a grid this small
    would only get the lower one)."""
    from gpt_fast_amd.ops import attention as A
    from gpt_fast_amd.ops import attention_bf16 as AB
    for row_tiles in ((1, 2) if dtype == torch.bfloat16 else (0,)):
        monkeypatch.setattr(AB, "TILED_ROW_TILES", row_tiles)
        _attention_over_pages(A, dtype, tol, H, G, hd, window)


def _attention_over_pages(A, dtype, tol, H, G, hd, window):
    lens = [1, 63, 64, 65, 200, 333]
    k_pages, v_pages, table, ks, vs = _paged(lens, G, hd, dtype, seed=hd + H)
    g = torch.Generator().manual_seed(5)
    tok_seq, tok_pos = [], []
    for b, S in enumerate(lens):
        new = list(range(S)) if b % 2 == 0 else [S - 1]        # whole prompt / one token
        tok_seq += [b] * len(new)
        tok_pos += new
    q = torch.randn(len(tok_seq), H, hd, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(hd)

    class B:
        pass
    batch = B()
    batch.tok_seq = torch.tensor(tok_seq, dtype=torch.int32, device=DEV)
    batch.tok_pos = torch.tensor(tok_pos, dtype=torch.int32, device=DEV)
    batch.n_tokens, batch.n_seqs = len(tok_seq), len(lens)
    batch.max_q_len, batch.max_kv_len, batch.is_decode = max(lens), max(lens), False
    starts = [0 if b % 2 == 0 else S - 1 for b, S in enumerate(lens)]
    qs = [0]
    for b, S in enumerate(lens):
        qs.append(qs[-1] + (S if b % 2 == 0 else 1))
    batch.q_start = torch.tensor(qs, dtype=torch.int32, device=DEV)
    batch.start_pos = torch.tensor(starts, dtype=torch.int32, device=DEV)
    batch.host_q_start, batch.host_start_pos = qs, starts
    out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, scale, window).cpu()
    plain = K().attention_generic(q.to(DEV), k_pages, v_pages, batch.tok_seq, batch.tok_pos,
                                  table, scale, window).cpu()
    assert not torch.isnan(out).any()
    for n in range(len(tok_seq)):
        b, p = tok_seq[n], tok_pos[n]
        ref = _attention_ref(q[n].float(), ks[b].float(), vs[b].float(), p, scale, window)
        close(out[n], ref, tol)
        close(plain[n], ref, tol)


@pytest.mark.parametrize("H,G,hd", [(4, 4, 16), (2, 2, 16), (6, 2, 32), (4, 4, 64), (8, 2, 128),
                                    (4, 2, 16), (3, 1, 48), (5, 5, 80), (4, 2, 256)])
def test_attention_of_a_chunk_at_an_offset(H, G, hd):
    """Several new tokens of a sequence whose first tokens are cached already (start
    position > 0), in row counts that take each form of the wave-level kernel (one, two and
    four row tiles per wave) and the workgroup-tiled one, over one and over several blocks
    of keys; pages beyond the newest key are poisoned."""
    from gpt_fast_amd.ops import attention as A
    scale = 1.0 / math.sqrt(hd)
    for spos, qlen in [(20, 20), (13, 20), (12, 20), (37, 29), (70, 5), (33, 17), (67, 33),
                       (100, 3), (1, 63), (130, 70)]:
        S = spos + qlen
        k_pages, v_pages, table, ks, vs = _paged([S], G, hd, torch.bfloat16, seed=spos + qlen)
        g = torch.Generator().manual_seed(5)
        q = torch.randn(qlen, H, hd, generator=g).to(torch.bfloat16)

        class B:
            pass
        batch = B()
        batch.tok_seq = torch.zeros(qlen, dtype=torch.int32, device=DEV)
        batch.tok_pos = torch.arange(spos, S, dtype=torch.int32, device=DEV)
        batch.n_tokens, batch.n_seqs = qlen, 1
        batch.max_q_len, batch.max_kv_len, batch.is_decode = qlen, S, False
        batch.q_start = torch.tensor([0, qlen], dtype=torch.int32, device=DEV)
        batch.start_pos = torch.tensor([spos], dtype=torch.int32, device=DEV)
        out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, scale, 0).cpu()
        assert not torch.isnan(out).any(), (spos, qlen)
        for n in range(qlen):
            ref = _attention_ref(q[n].float(), ks[0].float(), vs[0].float(), spos + n, scale, 0)
            close(out[n], ref, 1.5e-2)


def test_attention_finds_one_far_key():
    """One key among hundreds stands out (its score is scaled up): the output must be
    that key's value, wherever in the cache it lies - first row, a page edge, the last."""
    from gpt_fast_amd.ops import attention as A
    # 700 keys: six blocks per wave, no context split; 5000 keys: twenty splits, summed by
    # the second kernel in batches of eight and a rest; 9000 keys of a small head: thirty-two
    # splits, more than the lanes that hold the head's dims in that kernel; then other head
    # sizes and group sizes (two row tiles per kv head; two waves per workgroup) with splits
    cases = [(dtype, 700, t, 64, 4, 2) for dtype in (torch.float32, torch.bfloat16) for t in (0, 63, 64, 511, 699)]
    cases += [(torch.bfloat16, 5000, t, 64, 4, 2) for t in (0, 2047, 2600, 4999)]
    cases += [(torch.bfloat16, 9000, t, 32, 4, 2) for t in (100, 4400, 8999)]
    cases += [(torch.bfloat16, 3000, t, hd, H, G) for t in (5, 1500, 2999)
              for hd, H, G in ((256, 2, 1), (48, 6, 2), (128, 32, 1), (112, 5, 5))]
    for dtype, S, target, hd, H, G in cases:
        k_pages, v_pages, table, ks, vs = _paged([S], G, hd, dtype, seed=target)
        q = torch.zeros(1, H, hd)
        for h in range(H):
            q[0, h] = ks[0][target, h // (H // G)].float() * 40.0
        q = q.to(dtype)

        class B:
            pass
        batch = B()
        batch.tok_seq = torch.zeros(1, dtype=torch.int32, device=DEV)
        batch.tok_pos = torch.tensor([S - 1], dtype=torch.int32, device=DEV)
        batch.n_tokens = batch.n_seqs = 1
        batch.max_q_len, batch.max_kv_len, batch.is_decode = 1, S, True
        batch.q_start = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
        batch.start_pos = torch.tensor([S - 1], dtype=torch.int32, device=DEV)
        batch.host_q_start, batch.host_start_pos = [0, 1], [S - 1]
        out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, 1.0, 0).cpu().float()
        for h in range(H):
            close(out[0, h], vs[0][target, h // (H // G)].float(), 2e-2)


def _chunk_reference(q, k, v, spos, scale):
    """float64 attention of a chunk q [n, H, hd] at positions spos .. over k, v [S, G, hd]."""
    n, H, hd = q.shape
    S, G, _ = k.shape
    kk = k.double().repeat_interleave(H // G, dim=1)                 # [S, H, hd]
    vv = v.double().repeat_interleave(H // G, dim=1)
    s = torch.einsum("nhd,shd->hns", q.double(), kk) * scale
    mask = torch.arange(S)[None, :] > (spos + torch.arange(n))[:, None]
    s = s.masked_fill(mask[None], float("-inf"))
    return torch.einsum("hns,shd->nhd", torch.softmax(s, -1), vv)


@pytest.mark.parametrize("hd", [16, 32, 48, 64, 80, 96, 112, 128, 256])
def test_attention_variants_sweep(hd):
    """Every instantiation of the matrix-core attention, forced through the C entry points
    instead of chosen by shape: the wave-level kernel with one, two (the prefetching loop) and
    four row tiles per wave, one to four waves per workgroup and with the context split over
    workgroups; the workgroup-tiled kernel in both tile heights; chunks at an offset over one
    to five pages of keys; one and three query heads per kv head.  In every case some rows
    have a late key that stands out (a multiple of their own query), so that the running
    maximum moves - and the output accumulators are rescaled - in a block after the first;
    the comparison is with float64."""
    import ctypes
    from gpt_fast_amd.ops.library import library, ptr, stream_handle
    lib = library("attention_bf16")
    i32, f32 = ctypes.c_int, ctypes.c_float
    scale = 1.0 / math.sqrt(hd)
    for G, R in ((2, 1), (1, 3)):
        H = G * R
        for spos, qlen in [(0, 20), (13, 40), (70, 33), (100, 60), (250, 70)]:
            S = spos + qlen
            k_pages, v_pages, table, ks, vs = _paged([S], G, hd, torch.bfloat16, seed=hd + spos)
            gen = torch.Generator().manual_seed(spos + R)
            q = bf(torch.randn(qlen, H, hd, generator=gen))
            # every fourth token's first head of each group: its own position's key is three
            # times its query, the newest key it sees, in the last block it reads
            k_rows, v_cols = from_cache_order(k_pages.cpu(), v_pages.cpu())
            for n in range(1, qlen, 4):
                pos = spos + n
                page, off = int(table[0, pos // 64]), pos % 64
                for g in range(G):
                    ks[0][pos, g] = q[n, g * R] * 3.0
                    k_rows[page, g, off] = ks[0][pos, g]
            k_pages, _ = to_cache_order(k_rows, v_cols)
            k_pages = k_pages.to(DEV)
            want = _chunk_reference(q.float(), ks[0].float(), vs[0].float(), spos, scale)
            q_dev = q.to(DEV)
            q_start = torch.tensor([0, qlen], dtype=torch.int32, device=DEV)
            start = torch.tensor([spos], dtype=torch.int32, device=DEV)
            rows = qlen * R
            # waves that share a workgroup add their partial results in LDS: at most 64 KB
            per_wave = 128 + (2 if hd <= 64 else 4 if hd <= 128 else 8) * 2 * 1024
            cases = [("wave", rt, nw, sp) for rt in (1, 2, 4) for nw, sp in ((1, 1), (2, 1), (4, 3))
                     if not (rt == 4 and hd > 128) and (nw - 1) * rt * per_wave <= 65536]
            if hd <= 128:
                cases += [("tiled", rt, 4, 1) for rt in (1, 2)]
            for kind, rt, nw, splits in cases:
                out = torch.full((qlen, H, hd), float("nan"), dtype=torch.bfloat16, device=DEV)
                if kind == "tiled":
                    code = lib.gfa_attention_tiled_bf16(
                        ptr(q_dev), ptr(k_pages), ptr(v_pages), ptr(q_start), ptr(start), ptr(table),
                        i32(table.shape[1]), ptr(out), i32(qlen), i32(1), i32(H), i32(G), i32(hd),
                        f32(scale), i32(0), i32(rows), i32(rt), stream_handle())
                else:
                    ws_o = torch.empty((splits, qlen * H, hd), dtype=torch.float32, device=DEV)
                    ws_ml = torch.empty((splits, qlen * H, 2), dtype=torch.float32, device=DEV)
                    tiles = (rows + 16 * rt - 1) // (16 * rt)
                    code = lib.gfa_attention_bf16(
                        ptr(q_dev), ptr(k_pages), ptr(v_pages), ptr(q_start), ptr(start), ptr(table),
                        i32(table.shape[1]), ptr(out), ptr(ws_o), ptr(ws_ml), i32(qlen), i32(1),
                        i32(H), i32(G), i32(hd), f32(scale), i32(0), i32(rt), i32(nw), i32(tiles),
                        i32(splits), i32(0), i32(0), stream_handle())
                assert code == 0, (kind, rt, nw, splits, code)
                got = out.cpu().double()
                assert not torch.isnan(got).any(), (kind, rt, nw, splits, R, spos, qlen)
                err = float((got - want).abs().max() / want.abs().max())
                assert err < 1.5e-2, (kind, rt, nw, splits, R, spos, qlen, err)


@pytest.mark.parametrize("H,G,hd,window", [(8, 2, 128, 0), (4, 4, 16, 0), (16, 1, 64, 0), (6, 2, 48, 37),
                                           (3, 1, 256, 0), (10, 2, 112, 100), (32, 8, 128, 4000)])
def test_single_token_attention_in_a_batch(H, G, hd, window):
    """One new token for each sequence of a batch (the step that decoding repeats): lengths
    from one key to 4,100 in one launch - the last one's page row is longer than the 63
    entries a wave keeps in registers - on scattered pages with poisoned tails."""
    _single_token_batch(H, G, hd, window, [1, 63, 64, 65, 200, 333, 4100, 2])
    _single_token_batch(H, G, hd, window, [5, 333, 64, 129, 1])        # short: no context split
    _single_token_batch(H, G, hd, window, [3 + 11 * i for i in range(21)])    # rows chunked by 32
    _single_token_batch(H, G, hd, window, [70 - i for i in range(40)])        # and by 64


def _single_token_batch(H, G, hd, window, lens):
    from gpt_fast_amd.ops import attention as A
    from gpt_fast_amd.ops.gemm_bf16 import ChunkedRows
    k_pages, v_pages, table, ks, vs = _paged(lens, G, hd, torch.bfloat16, seed=hd + H)
    g = torch.Generator().manual_seed(6)
    q = torch.randn(len(lens), H, hd, generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(hd)

    class B:
        pass
    batch = B()
    batch.tok_seq = torch.arange(len(lens), dtype=torch.int32, device=DEV)
    batch.tok_pos = torch.tensor([S - 1 for S in lens], dtype=torch.int32, device=DEV)
    batch.n_tokens = batch.n_seqs = len(lens)
    batch.max_q_len, batch.max_kv_len, batch.is_decode = 1, max(lens), True
    batch.q_start = torch.arange(len(lens) + 1, dtype=torch.int32, device=DEV)
    batch.start_pos = batch.tok_pos.clone()
    batch.host_q_start, batch.host_start_pos = list(range(len(lens) + 1)), [S - 1 for S in lens]
    out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, scale, window).cpu()
    assert not torch.isnan(out).any()
    for b, S in enumerate(lens):
        ref = _attention_ref(q[b].float(), ks[b].float(), vs[b].float(), S - 1, scale, window)
        close(out[b], ref, 1.5e-2)
    # the same result in the order the output projection loads it in
    rows = A.attention(q.to(DEV), k_pages, v_pages, batch, table, scale, window, for_product=True)
    assert isinstance(rows, ChunkedRows) and rows.shape == (len(lens), H * hd)
    assert torch.equal(rows.to_rows().cpu().view(len(lens), H, hd), out)


@pytest.mark.parametrize("H,G,hd,window", [(8, 2, 128, 0), (4, 4, 64, 0), (6, 2, 96, 0), (8, 2, 128, 1000),
                                           (3, 1, 48, 0)])
def test_prompt_attention_over_thousands_of_keys(H, G, hd, window, monkeypatch):
    """The last 200 tokens of a 3000-token sequence as one prompt step: the workgroup-tiled
    kernel walks 47 pages per workgroup, in both its tile heights; every 13th row is compared
    with float64, and the last row must find one far key that stands out."""
    from gpt_fast_amd.ops import attention as A
    from gpt_fast_amd.ops import attention_bf16 as AB
    S, n_q, target = 3000, 200, 2345                      # inside the window of the last row
    k_pages, v_pages, table, ks, vs = _paged([S], G, hd, torch.bfloat16, seed=hd)
    g0 = torch.Generator().manual_seed(3)
    q = torch.randn(n_q, H, hd, generator=g0)
    for h in range(H):
        q[-1, h] = ks[0][target, h // (H // G)].float() * (40.0 * math.sqrt(hd))
    q = bf(q)
    scale = 1.0 / math.sqrt(hd)

    class B:
        pass
    batch = B()
    pos = list(range(S - n_q, S))
    batch.tok_seq = torch.zeros(n_q, dtype=torch.int32, device=DEV)
    batch.tok_pos = torch.tensor(pos, dtype=torch.int32, device=DEV)
    batch.n_tokens, batch.n_seqs = n_q, 1
    batch.max_q_len, batch.max_kv_len, batch.is_decode = n_q, S, False
    batch.q_start = torch.tensor([0, n_q], dtype=torch.int32, device=DEV)
    batch.start_pos = torch.tensor([S - n_q], dtype=torch.int32, device=DEV)
    batch.host_q_start, batch.host_start_pos = [0, n_q], [S - n_q]
    for row_tiles in (1, 2):
        monkeypatch.setattr(AB, "TILED_ROW_TILES", row_tiles)
        out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, scale, window).cpu().float()
        assert not torch.isnan(out).any()
        for n in list(range(0, n_q - 1, 13)):
            ref = _attention_ref(q[n].float(), ks[0].float(), vs[0].float(), pos[n], scale, window)
            close(out[n], ref, 1.5e-2)
        for h in range(H):
            close(out[-1, h], vs[0][target, h // (H // G)].float(), 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_query", [1, 40])
def test_attention_window_edge(dtype, n_query, monkeypatch):
    """A window of W keys: the key at distance W - 1 is the last one inside, the key at
    distance W the first one outside.  Two keys are made to stand out, one on each side of
    the edge of the last query: the output must be the inner one's value; with the outer
    one alone in sight of the score, it must not show.  One query row (the decode kernel)
    and forty (the prompt kernel)."""
    from gpt_fast_amd.ops import attention as A
    from gpt_fast_amd.ops import attention_bf16 as AB
    H, G, hd, S, W = 4, 2, 64, 333, 70
    both_heights = dtype == torch.bfloat16 and n_query > 1        # of the prompt kernel's tiles
    for inside, row_tiles in [(i, r) for i in (True, False) for r in ((1, 2) if both_heights else (0,))]:
        monkeypatch.setattr(AB, "TILED_ROW_TILES", row_tiles)
        k_pages, v_pages, table, ks, vs = _paged([S], G, hd, dtype, seed=17)
        last = S - 1
        edge_in, edge_out = last - W + 1, last - W
        target = edge_in if inside else edge_out
        q = torch.randn(n_query, H, hd) * 0.01
        for h in range(H):
            q[-1, h] = ks[0][target, h // 2].float() * 40.0
        q = q.to(dtype)

        class B:
            pass
        batch = B()
        pos = list(range(S - n_query, S))
        batch.tok_seq = torch.zeros(n_query, dtype=torch.int32, device=DEV)
        batch.tok_pos = torch.tensor(pos, dtype=torch.int32, device=DEV)
        batch.n_tokens, batch.n_seqs = n_query, 1
        batch.max_q_len, batch.max_kv_len, batch.is_decode = n_query, S, n_query == 1
        batch.q_start = torch.tensor([0, n_query], dtype=torch.int32, device=DEV)
        batch.start_pos = torch.tensor([S - n_query], dtype=torch.int32, device=DEV)
        batch.host_q_start, batch.host_start_pos = [0, n_query], [S - n_query]
        out = A.attention(q.to(DEV), k_pages, v_pages, batch, table, 1.0, W).cpu().float()
        for h in range(H):
            g = h // 2
            if inside:
                close(out[-1, h], vs[0][target, g].float(), 2e-2)
            else:
                # the outer key is masked: the row is an ordinary softmax over the window
                kk = ks[0][edge_in:last + 1, g].float()
                p = torch.softmax(kk @ q[-1, h].float(), 0)
                close(out[-1, h], p @ vs[0][edge_in:last + 1, g].float(), 3e-2)
                assert float((out[-1, h] - vs[0][target, g].float()).abs().max()) > 0.1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("H,G,hd,rot", [(4, 2, 16, 16), (3, 1, 48, 32), (2, 2, 128, 128)])
def test_rope_and_cache_write(dtype, layout, H, G, hd, rot):
    torch.manual_seed(6)
    pos = [0, 1, 63, 64, 130, 4000]
    N = len(pos)
    qkv = torch.randn(N, (H + 2 * G) * hd).to(dtype)
    freqs = 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))
    table = torch.tensor([[5, 3, 0, 1] + [2] * 60], dtype=torch.int32)
    k_pages = torch.zeros(6, G, 64, hd).to(dtype)
    v_pages = torch.zeros(6, G, hd, 64).to(dtype)
    kp, vp = k_pages.to(DEV), v_pages.to(DEV)
    q_out = K().rope_cache_write(
        qkv.to(DEV), freqs.to(DEV), torch.zeros(N, dtype=torch.int32, device=DEV),
        torch.tensor(pos, dtype=torch.int32, device=DEV), table.to(DEV), kp, vp, H, G, hd, rot,
        layout).cpu().float()
    x = qkv.float().reshape(N, H + 2 * G, hd)
    ang = torch.tensor(pos, dtype=torch.float32)[:, None] * freqs[None, :]
    c, s = torch.cos(ang.double())[:, None, :], torch.sin(ang.double())[:, None, :]
    ref = x.double().clone()
    qk = x[:, :H + G].double()
    if layout == 0:
        a, b = qk[..., 0:rot:2], qk[..., 1:rot:2]
        ref[:, :H + G, 0:rot:2] = a * c - b * s
        ref[:, :H + G, 1:rot:2] = b * c + a * s
    else:
        a, b = qk[..., :rot // 2], qk[..., rot // 2:rot]
        ref[:, :H + G, :rot // 2] = a * c - b * s
        ref[:, :H + G, rot // 2:rot] = b * c + a * s
    tol = 2e-4 if dtype == torch.float32 else 1e-2      # float: cos/sin of angles up to 4000
    close(q_out, ref[:, :H], tol)
    kc, vc = from_cache_order(kp.cpu().float(), vp.cpu().float())
    for n, p in enumerate(pos):
        page = int(table[0, p // 64])
        close(kc[page, :, p % 64], ref[n, H:H + G], tol)
        assert torch.equal(vc[page, :, :, p % 64], x[n, H + G:])
    # rotary_dim 0 and no pages: q passes through, nothing is written
    q2 = K().rope_cache_write(qkv.to(DEV), None, torch.zeros(N, dtype=torch.int32, device=DEV),
                              torch.tensor(pos, dtype=torch.int32, device=DEV), table.to(DEV),
                              None, None, H, G, hd, 0, 0).cpu()
    assert torch.equal(q2.reshape(N, -1), qkv[:, :H * hd])


@pytest.mark.parametrize("H,G,hd,rot,S", [(4, 2, 16, 16, 3), (3, 1, 48, 32, 1), (32, 8, 128, 128, 4), (2, 2, 32, 0, 5)])
def test_rope_and_cache_write_over_partial_sums(H, G, hd, rot, S):
    """The rotation and cache write that adds a sliced product's partial sums on its way:
    float partial sums [S, N, width] in, bfloat16 q and pages out, against float64 of the
    summed rows."""
    torch.manual_seed(16)
    pos = [0, 1, 63, 64, 130, 4000]
    N = len(pos)
    part = torch.randn(S, N, (H + 2 * G) * hd)
    freqs = 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / max(rot, 1)))
    table = torch.tensor([[5, 3, 0, 1] + [2] * 60], dtype=torch.int32)
    kp = torch.zeros(6, G, 64, hd, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(6, G, hd, 64, dtype=torch.bfloat16, device=DEV)
    q_out = K().rope_cache_write_sliced(
        part.to(DEV), freqs.to(DEV) if rot else None, torch.zeros(N, dtype=torch.int32, device=DEV),
        torch.tensor(pos, dtype=torch.int32, device=DEV), table.to(DEV), kp, vp, H, G, hd, rot).cpu()
    assert q_out.dtype == torch.bfloat16 and q_out.shape == (N, H, hd)
    x = part.double().sum(0).reshape(N, H + 2 * G, hd)
    ref = x.clone()
    if rot:
        ang = torch.tensor(pos, dtype=torch.float32)[:, None] * freqs[None, :]
        c, s = torch.cos(ang.double())[:, None, :], torch.sin(ang.double())[:, None, :]
        a, b = x[:, :H + G, 0:rot:2], x[:, :H + G, 1:rot:2]
        ref[:, :H + G, 0:rot:2] = a * c - b * s
        ref[:, :H + G, 1:rot:2] = b * c + a * s
    close(q_out, ref[:, :H], 1e-2)
    kc, vc = from_cache_order(kp.cpu().float(), vp.cpu().float())
    for n, p in enumerate(pos):
        page = int(table[0, p // 64])
        close(kc[page, :, p % 64], ref[n, H:H + G], 1e-2)
        close(vc[page, :, :, p % 64], ref[n, H + G:], 1e-2)


@pytest.mark.parametrize("window", [0, 50])
@pytest.mark.parametrize("H,G,hd,rot,S", [(32, 8, 128, 128, 4), (6, 2, 32, 16, 3), (4, 4, 64, 64, 1),
                                          (16, 1, 16, 0, 2), (12, 3, 48, 24, 2)])
def test_attention_over_partial_sums_of_the_projection(H, G, hd, rot, S, window):
    """One token per sequence, q, k and v still as the float partial sums of a sliced product:
    one kernel adds the slices, rotates, writes the new key and value to the cache and attends.
    Against float64 of the whole: the summed rows, rotated by interleaved pairs, the token's
    own key and value among the sequence's (contexts that end at a block's and a page's first
    and last places, long enough for context splits; dirty places behind the newest key)."""
    from gpt_fast_amd.ops import attention_bf16 as A
    torch.manual_seed(H + hd)
    ctx = [1, 32, 33, 64, 65, 200, 1000, 2049][:8]          # keys including the new one
    n = len(ctx)
    k_pages, v_pages, table, ks, vs = _paged(ctx, G, hd, torch.bfloat16, 5)
    part = torch.randn(S, n, (H + 2 * G) * hd)
    freqs = 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / max(rot, 1)))
    rows = part.double().sum(0).view(n, H + 2 * G, hd)
    pos = torch.tensor([c - 1 for c in ctx], dtype=torch.float32)
    ref = rows.clone()
    if rot:
        ang = pos[:, None] * freqs[None, :]
        c, s_ = torch.cos(ang.double())[:, None, :], torch.sin(ang.double())[:, None, :]
        a, b = rows[:, :H + G, 0:rot:2], rows[:, :H + G, 1:rot:2]
        ref[:, :H + G, 0:rot:2] = a * c - b * s_
        ref[:, :H + G, 1:rot:2] = b * c + a * s_
    q, k_new, v_new = ref[:, :H], ref[:, H:H + G], ref[:, H + G:]

    class Step:
        n_seqs, max_q_len = n, 1
        start_pos = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)

    kp, vp = k_pages.clone(), v_pages.clone()
    out = A.attention_sliced(part.to(DEV), freqs.to(DEV) if rot else None, rot, kp, vp, True, Step,
                             table, 1.0 / math.sqrt(hd), window, H)
    table, k_pages, v_pages = table.cpu(), k_pages.cpu(), v_pages.cpu()
    assert out is not None and out.shape == (n, H, hd)
    kc, vc = from_cache_order(kp.cpu().float(), vp.cpu().float())
    R = H // G
    for b_ in range(n):
        # the sequence's earlier keys and values as the cache holds them, the new ones as computed
        K_ = torch.cat([ks[b_][:ctx[b_] - 1].double(), k_new[b_][None]], 0)        # [ctx, G, hd]
        V_ = torch.cat([vs[b_][:ctx[b_] - 1].double(), v_new[b_][None]], 0)
        first = max(0, ctx[b_] - window) if window else 0     # keys at distance < window
        for h in range(H):
            g = h // R
            sc = (K_[first:, g] @ q[b_, h]) / math.sqrt(hd)
            want = torch.softmax(sc, 0) @ V_[first:, g]
            close(out[b_, h], want, 2e-2)
        page = int(table[b_, (ctx[b_] - 1) // 64])
        close(kc[page, :, (ctx[b_] - 1) % 64], k_new[b_], 1e-2)                  # written for later steps
        close(vc[page, :, :, (ctx[b_] - 1) % 64], v_new[b_], 1e-2)
    # nothing else in the cache changed
    k0, v0 = from_cache_order(k_pages.float(), v_pages.float())
    for b_ in range(n):
        page, off = int(table[b_, (ctx[b_] - 1) // 64]), (ctx[b_] - 1) % 64
        k0[page, :, off], v0[page, :, :, off] = kc[page, :, off], vc[page, :, :, off]
    assert torch.equal(torch.nan_to_num(k0, nan=7.0), torch.nan_to_num(kc, nan=7.0))
    assert torch.equal(torch.nan_to_num(v0, nan=7.0), torch.nan_to_num(vc, nan=7.0))


def test_argmax_and_sampling():
    from gpt_fast_amd.sampling import SamplingParams, logits_to_probs, sample
    import plain_llama as plain
    torch.manual_seed(7)
    B, V = 5, 1000
    logits = torch.randn(B, V, device=DEV) * 3
    logits[2, 17] = logits[2, 400] = 50.0                       # tie: the lowest index wins
    logits[3, 5] = float("nan")
    keys = torch.arange(B, dtype=torch.int32, device=DEV)
    got = K().argmax(logits).cpu()
    assert got[2] == 17
    clean = torch.nan_to_num(logits, nan=-1e30)
    assert torch.equal(got.long(), clean.argmax(-1).cpu())
    greedy = sample(logits, SamplingParams(temperature=0.0), keys, None)
    assert torch.equal(greedy.cpu(), got)

    logits = torch.randn(B, V, device=DEV) * 2
    for T, k in ((0.8, 50), (1.0, None), (0.3, 1), (1.5, 2000), (0.7, 7)):
        p = logits_to_probs(logits, T, k).cpu()
        ref = plain.logits_to_probs(logits.cpu(), T, k)
        assert torch.allclose(p, ref, rtol=1e-4, atol=1e-7), (T, k)
        if k is not None and k < V:
            assert ((p > 0).sum(-1) == k).all()
    top1 = sample(logits, SamplingParams(temperature=0.9, top_k=1, seed=3), keys, None)
    assert torch.equal(top1.cpu().long(), logits.argmax(-1).cpu())
    # ties with the k-th value survive
    tie = torch.zeros(1, 10, device=DEV)
    tie[0, :3] = 2.0
    tie[0, 3:6] = 1.0
    assert int((logits_to_probs(tie, 1.0, 4) > 0).sum()) == 6

    # frequencies follow the probabilities (chi-square, 3 degrees of freedom)
    small = torch.log(torch.tensor([[0.5, 0.25, 0.15, 0.1]], device=DEV)).repeat(4000, 1)
    rows = torch.arange(4000, dtype=torch.int32, device=DEV)
    draws = sample(small, SamplingParams(temperature=1.0, seed=11), rows, None).cpu()
    counts = torch.bincount(draws.long(), minlength=4).double()
    expect = torch.tensor([0.5, 0.25, 0.15, 0.1]).double() * 4000
    assert float(((counts - expect) ** 2 / expect).sum()) < 16.3      # p = 0.001

    # a row's draw depends on (seed, key, position) only, not on its place in the batch
    params = SamplingParams(temperature=1.0, top_k=100, seed=5)
    pos = torch.tensor([4, 9, 2, 7, 7], dtype=torch.int32, device=DEV)
    a = sample(logits, params, keys, pos, 1).cpu()
    order = torch.tensor([3, 0, 4, 2, 1], device=DEV)
    b = sample(logits[order].contiguous(), params, keys[order].contiguous(),
               pos[order].contiguous(), 1).cpu()
    assert torch.equal(b, a[order.cpu()])
    c = sample(logits, SamplingParams(temperature=1.0, top_k=100, seed=6), keys, pos, 1).cpu()
    assert not torch.equal(a, c)


@pytest.mark.parametrize("M", [1, 2, 5, 16, 17, 20, 21, 24, 25, 31, 33, 48, 64])
@pytest.mark.parametrize("D,K_,N2,eps", [(72, 40, 48, 1e-5), (200, 328, 208, 1e-6),
                                         (4096, 1024, 256, 1e-5), (1000, 64, 96, 0.3),
                                         (8192, 64, 64, 1e-5)])
def test_norm_over_two_kernels(M, D, K_, N2, eps):
    """The product that completes the residual stream prepares the next norm (column
    weights applied, shares of the sums of squares); the next product applies the row
    factor.  Against float64, and against the engine's own separate kernels."""
    from gpt_fast_amd.ops import gemm_bf16 as G
    torch.manual_seed(10)
    res0 = torch.randn(M, D, device=DEV) * 3
    res0[0] *= 50.0                                   # rows of very different size
    y = bf(torch.randn(M, K_, device=DEV))
    wo = bf(torch.randn(D, K_, device=DEV) * 0.2)
    g = 1 + 0.1 * torch.randn(D, device=DEV)
    w = bf(torch.randn(N2, D, device=DEV) * 0.1)
    res = res0.clone()
    xg, ssq = G.skinny_into_chain(y, wo, res, g)
    res_ref = res0.double() + y.double() @ wo.double().T
    close(res, res_ref, 1e-5)
    close(ssq.sum(0)[:M], (res.double() ** 2).sum(1), 1e-5)
    assert ssq.shape[1] == (4 if M <= 4 else 8 if M <= 8 else 16 if M <= 16 else 32 if M <= 32 else 64)
    assert M == ssq.shape[1] or float(ssq[:, M:].abs().max()) == 0
    n = res.double() * torch.rsqrt((res.double() ** 2).mean(-1, keepdim=True) + eps) * g.double()
    ref = n @ w.double().T
    close(G.skinny_after_chain(xg, ssq, eps, w, out_dtype=torch.float32), ref, 1e-2)
    close(G.skinny_after_chain(xg, ssq, eps, w), ref, 1.5e-2)
    I = N2 // 2
    a = ref[:, :I]
    close(G.skinny_after_chain_gated(xg, ssq, eps, w), (a * torch.sigmoid(a)) * ref[:, I:], 2e-2)
    separate = G.skinny(K().rmsnorm(res, g, eps, torch.bfloat16), w, out_dtype=torch.float32)
    close(G.skinny_after_chain(xg, ssq, eps, w, out_dtype=torch.float32), separate, 1e-2)
    # row by row: a row's factor must be its own
    got = G.skinny_after_chain(xg, ssq, eps, w, out_dtype=torch.float32).double().cpu()
    for m in range(M):
        assert float((got[m] - ref[m].cpu()).abs().max() / ref[m].abs().max()) < 1.5e-2
    # the two halves put together by hand are the norm's rows
    rs = torch.rsqrt(ssq.sum(0)[:M, None].double() / D + eps)
    close(xg.to_rows().double() * rs, n, 1e-2)
    # the gate's result left in the order the next product loads it in: the same values, and
    # the same product from them
    if I % 8 == 0:
        h_rows = G.skinny_after_chain_gated(xg, ssq, eps, w)
        h_chunked = G.skinny_after_chain_gated(xg, ssq, eps, w, chunked=True)
        assert torch.equal(h_chunked.to_rows(), h_rows)
        w2 = bf(torch.randn(D, I, device=DEV) * 0.2)
        res_a, res_b = res0.clone(), res0.clone()
        xg_a, ssq_a = G.skinny_into_chain(h_rows, w2, res_a, g)
        xg_b, ssq_b = G.skinny_into_chain(h_chunked, w2, res_b, g)
        assert torch.equal(res_a, res_b) and torch.equal(ssq_a, ssq_b)
        assert torch.equal(xg_a.to_rows(), xg_b.to_rows())


@pytest.mark.parametrize("M", [9, 12, 16, 18, 20, 23, 24, 32, 40, 48])
def test_wide_matrices_at_nine_to_sixteen_rows(M):
    """From 6,144 rows of W on, a workgroup of the few-row kernel takes two tiles of W against
    the same fragments of x (nine to 48 rows of x): every epilogue on such a shape, the
    last workgroup with a second tile that is partly or wholly beyond the matrix."""
    from gpt_fast_amd.ops import gemm_bf16 as G
    torch.manual_seed(M)
    K_ = 264
    for N in (6144, 8200, 8216):
        x = bf(torch.randn(M, K_, device=DEV))
        w = bf(torch.randn(N, K_, device=DEV) * 0.1)
        ref = x.double() @ w.double().T
        close(G.skinny(x, w, out_dtype=torch.float32), ref, 1e-5)
        close(G.skinny(x, w), ref, 1e-2)
        res0 = torch.randn(M, N, device=DEV)
        res = res0.clone()
        G.skinny(x, w, residual=res)
        close(res, res0.double() + ref, 1e-5)
        # the norm in two halves: produced on the wide shape, consumed by a wide shape
        g = 1 + 0.1 * torch.randn(N, device=DEV)
        res = res0.clone()
        xg, ssq = G.skinny_into_chain(x, w, res, g)
        new = res0.double() + ref
        close(res, new, 1e-5)
        close(ssq.sum(0)[:M], (new ** 2).sum(1), 1e-5)
        eps = 1e-5
        n = new * torch.rsqrt((new ** 2).mean(-1, keepdim=True) + eps) * g.double()
        close(xg.to_rows().double() * torch.rsqrt(ssq.sum(0)[:M, None].double() / N + eps), n, 1e-2)
        w2 = bf(torch.randn(8192 + 16, N, device=DEV) * 0.02)
        close(G.skinny_after_chain(xg, ssq, eps, w2, out_dtype=torch.float32), n @ w2.double().T, 1e-2)
    # the gate: two tiles of W1's rows and their two tiles of W3's rows per workgroup (9..16 rows)
    for I in (6144, 6152):
        x = bf(torch.randn(M, K_, device=DEV))
        w13 = bf(torch.randn(2 * I, K_, device=DEV) * 0.1)
        a = x.double() @ w13.double().T
        close(G.skinny_gated(x, w13), (a[:, :I] * torch.sigmoid(a[:, :I])) * a[:, I:], 2e-2)
    # projection, rotation and cache write: 64 heads of 128 are 8,192 rows of W
    H, G_, hd = 48, 8, 128
    tok_seq = torch.arange(M, dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor([5 + 5 * i for i in range(M)], dtype=torch.int32, device=DEV)
    assert int(tok_pos.max()) < 4 * 64                     # four pages per sequence
    table = torch.arange(M * 4, dtype=torch.int32, device=DEV).view(M, 4)
    freqs = (1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))).to(DEV)
    xn = bf(torch.randn(M, K_, device=DEV))
    wq = bf(torch.randn((H + 2 * G_) * hd, K_, device=DEV) * 0.1)
    kp = torch.zeros(M * 4, G_, 64, hd, device=DEV, dtype=torch.bfloat16)
    vp = torch.zeros(M * 4, G_, hd, 64, device=DEV, dtype=torch.bfloat16)
    q = G.qkv_rope_store(xn, wq, freqs, tok_seq, tok_pos, table, kp, vp, H, G_, hd, hd)
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    q2 = K().rope_cache_write(G.skinny(xn, wq), freqs, tok_seq, tok_pos, table, kp2, vp2, H, G_, hd, hd, 0)
    close(q, q2, 1e-2)
    close(kp, kp2, 1e-2)
    assert torch.equal(vp, vp2)
    assert torch.equal(kp == 0, kp2 == 0) and torch.equal(vp == 0, vp2 == 0)
    # and against float64 of the whole: product, rotation by interleaved pairs, the page and
    # place each token's keys and values went to
    rows = (xn.double() @ wq.double().T).view(M, H + 2 * G_, hd).cpu()
    ang = tok_pos.cpu().float()[:, None] * freqs.cpu()[None, :]
    c, s_ = torch.cos(ang.double())[:, None, :], torch.sin(ang.double())[:, None, :]
    ref = rows.clone()
    a, b = rows[:, :H + G_, 0::2], rows[:, :H + G_, 1::2]
    ref[:, :H + G_, 0::2] = a * c - b * s_
    ref[:, :H + G_, 1::2] = b * c + a * s_
    close(q, ref[:, :H], 1e-2)
    kc, vc = from_cache_order(kp.cpu().float(), vp.cpu().float())
    for n in range(M):
        p_ = int(tok_pos[n])
        close(kc[4 * n + p_ // 64, :, p_ % 64], ref[n, H:H + G_], 1e-2)
        close(vc[4 * n + p_ // 64, :, :, p_ % 64], ref[n, H + G_:], 1e-2)


@pytest.mark.parametrize("H,G_,hd,rot", [(4, 2, 16, 16), (3, 1, 48, 32), (32, 8, 128, 128), (2, 2, 32, 0)])
def test_projection_rotation_and_cache_write_in_one_kernel(H, G_, hd, rot):
    from gpt_fast_amd.ops import gemm_bf16 as G
    torch.manual_seed(9)
    D = 72 if hd < 128 else 512
    pos = [0, 5, 63, 64, 200, 3000]
    seq = [1, 0, 1, 0, 1, 0]                      # two sequences with tables of their own
    M = len(pos)
    x = torch.randn(M, D, device=DEV)
    g = 1 + 0.1 * torch.randn(D, device=DEV)
    w = bf(torch.randn((H + 2 * G_) * hd, D, device=DEV) * 0.1)
    freqs = (1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV) if rot else None
    table = torch.stack([torch.randperm(50)[:48], torch.randperm(50)[:48] + 50]).to(torch.int32).to(DEV)
    tok_seq = torch.tensor(seq, dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor(pos, dtype=torch.int32, device=DEV)
    kp = torch.zeros(100, G_, 64, hd, device=DEV, dtype=torch.bfloat16)
    vp = torch.zeros(100, G_, hd, 64, device=DEV, dtype=torch.bfloat16)
    xn = K().rmsnorm(x, g, 1e-5, torch.bfloat16)
    q = G.qkv_rope_store(xn, w, freqs, tok_seq, tok_pos, table, kp, vp, H, G_, hd, rot)
    # the separate kernels of the same engine
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    qkv = G.skinny(xn, w)
    q2 = K().rope_cache_write(qkv, freqs, tok_seq, tok_pos, table, kp2, vp2, H, G_, hd, rot, 0)
    close(q, q2, 1e-2)
    close(kp, kp2, 1e-2)
    assert torch.equal(vp, vp2)                        # values are not rotated: same products
    assert torch.equal(kp == 0, kp2 == 0) and torch.equal(vp == 0, vp2 == 0)   # same places written
    # and a reference of their own, in float64: the product of the normed rows, rotated by
    # interleaved pairs (model.py:284-292), read back from the pages the table names
    rows = (xn.double() @ w.double().T).view(M, H + 2 * G_, hd).cpu()
    ref = rows.clone()
    if rot:
        ang = torch.tensor(pos, dtype=torch.float32)[:, None] * freqs.cpu()[None, :]
        c, s_ = torch.cos(ang.double())[:, None, :], torch.sin(ang.double())[:, None, :]
        a, b = rows[:, :H + G_, 0:rot:2], rows[:, :H + G_, 1:rot:2]
        ref[:, :H + G_, 0:rot:2] = a * c - b * s_
        ref[:, :H + G_, 1:rot:2] = b * c + a * s_
    close(q, ref[:, :H], 1e-2)
    kc, vc = from_cache_order(kp.cpu().float(), vp.cpu().float())
    written = torch.zeros(100, 64, dtype=torch.bool)
    for n in range(M):
        page = int(table[seq[n], pos[n] // 64])
        written[page, pos[n] % 64] = True
        close(kc[page, :, pos[n] % 64], ref[n, H:H + G_], 1e-2)
        close(vc[page, :, :, pos[n] % 64], ref[n, H + G_:], 1e-2)
    assert not kc.permute(0, 2, 1, 3)[~written].any() and not vc.permute(0, 3, 1, 2)[~written].any()
    # no pages: q only
    q3 = G.qkv_rope_store(xn, w, freqs, tok_seq, tok_pos, table, None, None, H, G_, hd, rot)
    assert torch.equal(q3, q)
    # rows whose norm arrives in two halves
    if D % 8 == 0:
        y = bf(torch.randn(M, 64, device=DEV))
        wo = bf(torch.randn(D, 64, device=DEV) * 0.2)
        res = x.clone()
        xg, ssq = G.skinny_into_chain(y, wo, res, g)
        kp5, vp5 = torch.zeros_like(kp), torch.zeros_like(vp)
        q5 = G.qkv_rope_store(xg, w, freqs, tok_seq, tok_pos, table, kp5, vp5, H, G_, hd, rot,
                              ssq=ssq, eps=1e-5)
        kp6, vp6 = torch.zeros_like(kp), torch.zeros_like(vp)
        q6 = G.qkv_rope_store(K().rmsnorm(res, g, 1e-5, torch.bfloat16), w, freqs, tok_seq, tok_pos,
                              table, kp6, vp6, H, G_, hd, rot)
        close(q5, q6, 1.5e-2)
        close(kp5, kp6, 1.5e-2)
        close(vp5, vp6, 1.5e-2)


def test_sampling_over_many_workgroups_equals_one_workgroup():
    """Large vocabularies are spread over many workgroups per row; the choice, the
    probabilities and the draws must be those of the one-workgroup kernels."""
    from gpt_fast_amd.ops import kernels as KK
    from gpt_fast_amd.sampling import SamplingParams, logits_to_probs, sample
    torch.manual_seed(10)
    B, V = 6, 50001                                     # no multiple of the chunk or of 4
    logits = torch.randn(B, V, device=DEV) * 3
    logits[1, 40000] = logits[1, 123] = 30.0            # a tie across chunks: lowest index
    logits[2, 7] = float("nan")
    keys = torch.arange(B, dtype=torch.int32, device=DEV)
    pos = torch.tensor([3, 1, 4, 1, 5, 9], dtype=torch.int32, device=DEV)
    results = {}
    for limit in (10 ** 9, 1000):                       # one workgroup per row / split
        KK.SPLIT_SAMPLING_ABOVE = limit
        try:
            r = [KK.argmax(logits).cpu()]
            for T, k in ((0.8, 200), (1.0, None), (0.5, 1), (1.3, 5000)):
                r.append(sample(logits, SamplingParams(T, k, 11), keys, pos, 1).cpu())
                r.append(logits_to_probs(logits, T, k).cpu())
            results[limit] = r
        finally:
            KK.SPLIT_SAMPLING_ABOVE = 16384
    one, split = results[10 ** 9], results[1000]
    assert int(one[0][1]) == 123 and torch.equal(one[0], split[0])
    for a, b in zip(one[1:], split[1:]):
        if a.dtype == torch.int32:
            assert torch.equal(a, b)
        else:
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-9)
            assert torch.equal(a > 0, b > 0)            # the same entries are kept
