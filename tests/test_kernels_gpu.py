"""Each HIP kernel alone against a plain torch reference, at sizes of its own."""

import math

import pytest
import torch

import plain_gpt2 as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _k():
    from mlx_lm_amd.ops import kernels

    return kernels


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


# ---------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 1600, 200])
def test_embed_gather_add(dtype, width):
    k = _k()
    V, P, T = 301, 77, 53
    table = _rand((V, width), dtype, 1)
    pos_table = _rand((P, width), dtype, 2)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32).to(DEV)
    pos = torch.randint(0, P, (T,), generator=g, dtype=torch.int32).to(DEV)
    out = torch.empty(T, width, dtype=torch.float32, device=DEV)
    k.embed_gather_add(out, table, ids, pos_table, pos)
    want = table.float()[ids.long()] + pos_table.float()[pos.long()]
    assert torch.equal(out, want)
    k.embed_gather_add(out, table, ids)
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,eps", [(64, 1e-5), (1600, 1e-6), (200, 1e-3), (198, 1e-5), (4096, 1e-5), (4104, 1e-5)])
def test_layernorm(out_dtype, width, eps):
    k = _k()
    R = 37
    x = _rand((R, width), torch.float32, 4, 3.0) + 1.5
    x[5] = x[5] * 1e-3  # a low-variance row, where eps matters
    gamma = 1 + _rand((width,), torch.float32, 5, 0.1)
    beta = _rand((width,), torch.float32, 6, 0.1)
    out = torch.empty(R, width, dtype=out_dtype, device=DEV)
    k.layernorm(out, x, gamma, beta, eps)
    want = plain.layer_norm(x.double().cpu(), gamma.double().cpu(), beta.double().cpu(), eps)
    tol = 2e-5 if out_dtype == torch.float32 else 2e-2
    assert torch.allclose(out.double().cpu(), want, atol=tol, rtol=tol)
    # gathered rows
    rows = torch.tensor([7, 0, 36, 7], dtype=torch.int32, device=DEV)
    out2 = torch.empty(4, width, dtype=out_dtype, device=DEV)
    k.layernorm(out2, x, gamma, beta, eps, rows=rows)
    assert torch.equal(out2, out[rows.long()])


GEMM_SHAPES = [
    (1, 48, 64),
    (3, 50, 1608),
    (8, 1600, 6400),
    (7, 1000, 96),
    (16, 80, 200),
    (33, 257, 384),
    (64, 4800, 1600),
    (130, 300, 72),
    (300, 513, 1608),
    (700, 520, 200),
    (130, 48, 16),  # K shorter than a k-block of the tile kernels
    (100, 96, 32),
    (70, 100, 48),
    (2100, 2064, 136),  # 17 x 17 tiles of 128: more blocks than CUs, two to a CU
]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("mode", ["plain", "gelu", "accumulate"])
def test_gemm_f32(M, N, K, mode):
    k = _k()
    a = _rand((M, K), torch.float32, 10)
    w = _rand((N, K), torch.float32, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    for variant in (1, 2, 3) if M <= 64 else (1, 2):  # tiles of 128 and of 64, the kernel for few rows
        if mode == "accumulate":
            out = _rand((M, N), torch.float32, 13)
            want = out.double().cpu() + ref
            k.linear(out, a, w, bias, accumulate=True, variant=variant)
        else:
            out = torch.empty(M, N, dtype=torch.float32, device=DEV)
            k.linear(out, a, w, bias, gelu=(mode == "gelu"), variant=variant)
            want = plain.gelu_tanh(ref) if mode == "gelu" else ref
        err = (out.double().cpu() - want).abs().max().item()
        assert err < 1e-5 * math.sqrt(K) * 4, (variant, err)


@pytest.mark.parametrize("N,K", [(1, 4), (7, 508), (9, 512), (17, 516), (40, 1024), (33, 1028), (100, 1600),
                                 (24, 2052), (4100, 520), (4097, 1600)])
def test_gemm_f32_few_rows(N, K):
    """The kernel for up to 64 rows at the edges of its chunks of 64 columns, of a block's 16
    features and of its blocks of 16 rows, with 8 and with 4 waves a block (from 4,096 features on
    there is a block for every compute unit), with K whole and in parts, and that a row's result
    does not depend on how many other rows the step holds."""
    k = _k()
    w = _rand((N, K), torch.float32, 21, 0.1)
    bias = _rand((N,), torch.float32, 22)
    a_all = _rand((64, K + 4), torch.float32, 23)[:, :K]  # rows with a stride of their own
    alone = torch.empty(1, N, dtype=torch.float32, device=DEV)
    k.linear(alone, a_all[:1], w, bias, variant=3)
    for M in (1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 47, 49, 64):
        a = a_all[:M]
        wide = torch.full((M, N + 3), float("nan"), dtype=torch.float32, device=DEV)
        out = wide[:, :N]
        k.linear(out, a, w, bias, variant=3)
        ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
        err = (out.double().cpu() - ref).abs().max().item()
        assert err < 1e-5 * math.sqrt(K) * 4, (M, err)
        assert torch.isnan(wide[:, N:]).all()
        assert torch.equal(out[:1], alone), M
        k.linear(out, a, w, None, accumulate=True, variant=3)
        err = (out.double().cpu() - (2 * ref - bias.double().cpu())).abs().max().item()
        assert err < 2e-5 * math.sqrt(K) * 4, (M, err)
        # K in parts over the blocks, added up by the second kernel
        for splits in (2, 3, 7):
            for mode in ("plain", "gelu", "accumulate"):
                got = torch.full((M, N), 0.5, dtype=torch.float32, device=DEV)
                k.linear(got, a, w, bias, gelu=(mode == "gelu"), accumulate=(mode == "accumulate"), variant=3,
                         splits=splits)
                want = {"plain": ref, "gelu": plain.gelu_tanh(ref), "accumulate": ref + 0.5}[mode]
                err = (got.double().cpu() - want).abs().max().item()
                assert err < 1e-5 * math.sqrt(K) * 4, (M, splits, mode, err)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("mode", ["plain", "gelu", "accumulate", "f32out"])
def test_gemm_bf16(M, N, K, mode):
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    variants = (1, 2, 3, 4, 5, 6, 7) if M <= 64 else (1, 3, 4, 5, 6, 7)  # tiles of 128 x 128, skinny, 256 x 256, 256 x 192, 64 x 128, 32 x 128, 128 x 128 with eight waves
    for variant in variants:
        if mode == "accumulate":
            out = _rand((M, N), torch.float32, 13)
            want = out.double().cpu() + ref
            k.linear(out, a, w, bias, accumulate=True, variant=variant)
            tol = 1e-4 * math.sqrt(K)
        elif mode == "f32out":
            out = torch.empty(M, N, dtype=torch.float32, device=DEV)
            k.linear(out, a, w, bias, variant=variant)
            want = ref
            tol = 1e-4 * math.sqrt(K)
        else:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            k.linear(out, a, w, bias, gelu=(mode == "gelu"), variant=variant)
            want = plain.gelu_tanh(ref) if mode == "gelu" else ref
            tol = None
        got = out.double().cpu()
        if tol is None:
            # one bfloat16 rounding of the exact value
            assert torch.allclose(got, want, rtol=2**-7, atol=1e-3), (variant, (got - want).abs().max())
        else:
            assert (got - want).abs().max().item() < tol, (variant, (got - want).abs().max())


def test_gemm_refuses_bad_sizes():
    k = _k()
    a = torch.zeros(4, 20, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 20, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(4, 8, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        k.linear(out, a, w)
    with pytest.raises(ValueError):
        k.linear(out, a.float(), w)


# ---------------------------------------------------------------------------
# paged attention


class PagedCase:
    """Random requests with a scrambled page assignment and a ragged step."""

    def __init__(self, dtype, n_heads, n_kv_heads, head_dim, page_size, ctx_lens, q_lens, seed,
                 window=0):
        from mlx_lm_amd.ops.kernels import PagedKV

        g = torch.Generator().manual_seed(seed)
        self.dtype, self.H, self.Hkv, self.hd, self.ps = dtype, n_heads, n_kv_heads, head_dim, page_size
        self.window = window
        R = len(ctx_lens)
        self.total = [c + q for c, q in zip(ctx_lens, q_lens)]
        max_blocks = max((t + page_size - 1) // page_size for t in self.total) + 1
        n_pages = sum((t + page_size - 1) // page_size for t in self.total) + 3
        perm = torch.randperm(n_pages, generator=g).tolist()
        self.block_table = torch.full((R, max_blocks), -1, dtype=torch.int32)
        pool = torch.full((n_pages, 2, n_kv_heads, page_size, head_dim), float("nan")).to(dtype)
        self.k_full, self.v_full = [], []
        nxt = 0
        for r in range(R):
            kf = torch.randn(self.total[r], n_kv_heads, head_dim, generator=g).to(dtype)
            vf = torch.randn(self.total[r], n_kv_heads, head_dim, generator=g).to(dtype)
            self.k_full.append(kf)
            self.v_full.append(vf)
            for b in range((self.total[r] + page_size - 1) // page_size):
                self.block_table[r, b] = perm[nxt]
                nxt += 1
            # tokens already in the cache; this step's tokens go through kv_write
            for p in range(ctx_lens[r]):
                page = self.block_table[r, p // page_size]
                pool[page, 0, :, p % page_size] = kf[p]
                pool[page, 1, :, p % page_size] = vf[p]
        self.pool = pool.to(DEV)
        self.kv = PagedKV(self.pool[:, 0], self.pool[:, 1])
        token_req, positions = [], []
        for r in range(R):
            for i in range(q_lens[r]):
                token_req.append(r)
                positions.append(ctx_lens[r] + i)
        self.T = len(token_req)
        self.token_req = torch.tensor(token_req, dtype=torch.int32, device=DEV)
        self.positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
        self.q = torch.randn(self.T, n_heads * head_dim, generator=g).to(dtype)
        self.k_new = torch.stack([self.k_full[r][p] for r, p in zip(token_req, positions)]).reshape(self.T, -1)
        self.v_new = torch.stack([self.v_full[r][p] for r, p in zip(token_req, positions)]).reshape(self.T, -1)
        self.block_table_dev = self.block_table.to(DEV)
        self.ctx_lens, self.q_lens = ctx_lens, q_lens
        self.scale = head_dim**-0.5

    def reference(self):
        out = torch.empty(self.T, self.H * self.hd, dtype=torch.float64)
        t = 0
        for r, (c, n) in enumerate(zip(self.ctx_lens, self.q_lens)):
            if n == 0:
                continue
            q = self.q[t : t + n].double().reshape(n, self.H, self.hd).permute(1, 0, 2)
            kk = self.k_full[r][: c + n].double().permute(1, 0, 2)
            vv = self.v_full[r][: c + n].double().permute(1, 0, 2)
            mask = plain.causal_mask(n, c, self.window if self.window else None)
            o = plain.attention(q, kk, vv, self.scale, mask)
            out[t : t + n] = plain.merge_heads(o)
            t += n
        return out

    def tiles(self, qt=16):
        tiles, t = [], 0
        for n in self.q_lens:
            for s in range(0, n, qt):
                tiles.append((t + s, min(qt, n - s)))
            t += n
        return torch.tensor(tiles, dtype=torch.int32, device=DEV)


ATTN_CASES = [
    # H, Hkv, hd, page, ctx_lens, q_lens, window
    (4, 4, 16, 16, [0, 5, 40], [33, 1, 7], 0),
    (3, 3, 32, 16, [0, 100, 17, 64], [90, 1, 2, 1], 0),
    (6, 2, 48, 8, [3, 0, 250], [20, 70, 1], 0),
    (5, 1, 80, 32, [130, 0], [1, 130], 0),
    (2, 2, 128, 64, [200, 0], [3, 65], 0),
    (4, 2, 64, 16, [0, 300, 90], [200, 1, 5], 37),
    (25, 25, 64, 16, [511, 0], [1, 48], 0),
]


def _attn_tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.6e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_kv_write_and_attn_tile(dtype, case):
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(dtype, H, Hkv, hd, ps, ctx, ql, seed=hd + H, window=window)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    torch.cuda.synchronize()
    # every written token is where the table says, bit for bit
    pool = c.pool.cpu()
    for r in range(len(ctx)):
        for p in range(c.total[r]):
            page = c.block_table[r, p // ps]
            assert torch.equal(pool[page, 0, :, p % ps], c.k_full[r][p])
            assert torch.equal(pool[page, 1, :, p % ps], c.v_full[r][p])
    tiles = c.tiles()
    out = torch.full((c.T, H * hd), float("nan")).to(dtype).to(DEV)
    k.attn_tile(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, tiles,
                tiles.shape[0], H, c.scale, window)
    want = c.reference()
    err = (out.double().cpu() - want).abs().max().item()
    assert err < _attn_tol(dtype), err


@pytest.mark.parametrize("case", [
    # H, Hkv, hd, page, ctx_lens, q_lens, window
    (3, 3, 64, 16, [0, 100, 17, 64, 15], [90, 1, 2, 17, 16], 0),
    (6, 2, 64, 48, [3, 0, 250], [20, 70, 1], 0),
    (5, 1, 128, 32, [130, 0, 31], [1, 130, 34], 0),
    (4, 2, 64, 16, [0, 300, 90], [200, 1, 5], 37),
    (2, 2, 128, 16, [0, 300], [150, 33], 16),
    (2, 1, 64, 32, [500, 0], [40, 300], 1),
])
def test_attn_tile_float32_on_matrix_cores(case):
    """Float caches with head_dim 64 or 128 in pages of whole 16 keys: a wave a tile of 16 queries
    and 16 keys at a time; tiles that start and end inside a page, short last tiles, windows that
    end inside a tile of keys, grouped heads.  Free page slots hold NaN."""
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(torch.float32, H, Hkv, hd, ps, ctx, ql, seed=hd + H + ps, window=window)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    tiles = c.tiles()
    out = torch.full((c.T, H * hd), float("nan"), dtype=torch.float32, device=DEV)
    k.attn_tile(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, tiles,
                tiles.shape[0], H, c.scale, window)
    err = (out.double().cpu() - c.reference()).abs().max().item()
    assert err < _attn_tol(torch.float32), err


def test_attn_tile_float32_far_key_stands_out():
    """A prompt's last query points at one key among hundreds: a dropped or doubled tile of keys shows."""
    k = _k()
    H, hd, ps = 2, 64, 16
    for far in (0, 3, 4, 15, 16, 17, 255, 256, 383, 384, 399):
        c = PagedCase(torch.float32, H, H, hd, ps, [0], [400], seed=far)
        kf = c.k_full[0][far, 1].clone()
        c.q[399, hd:] = kf * (30.0 / (c.scale * float(kf.norm() ** 2)))
        k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
        tiles = c.tiles()
        out = torch.full((c.T, H * hd), float("nan"), dtype=torch.float32, device=DEV)
        k.attn_tile(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, tiles,
                    tiles.shape[0], H, c.scale, 0)
        assert (out[399, hd:].double().cpu() - c.v_full[0][far, 1].double()).abs().max().item() < 0.1, far
        assert (out.double().cpu() - c.reference()).abs().max().item() < _attn_tol(torch.float32), far


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kv_write_from_rows_that_are_not_aligned(dtype):
    """Sources that start in the middle of a 16-byte piece take the element-wise kernel: same pages."""
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = ATTN_CASES[0]
    c = PagedCase(dtype, H, Hkv, hd, ps, ctx, ql, seed=3, window=window)
    start = c.pool.clone()  # (holds the keys and values of the tokens before)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    want = c.pool.clone()
    bits = torch.int32 if dtype == torch.float32 else torch.int16  # (free slots hold NaN: compare bits)
    assert not torch.equal(want.view(bits), start.view(bits))
    c.pool.copy_(start)
    width = c.k_new.shape[1]
    wide = torch.zeros(c.T, 2 * width + 8, dtype=dtype, device=DEV)
    wide[:, 1 : 1 + width] = c.k_new.to(DEV)
    wide[:, 1 + width : 1 + 2 * width] = c.v_new.to(DEV)
    k.kv_write(wide[:, 1 : 1 + width], wide[:, 1 + width : 1 + 2 * width], c.kv, c.block_table_dev, c.token_req,
               c.positions)
    assert torch.equal(c.pool.view(bits), want.view(bits))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTN_CASES)
@pytest.mark.parametrize("n_splits", [1, 3, 8])
def test_attn_row(dtype, case, n_splits):
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(dtype, H, Hkv, hd, ps, ctx, ql, seed=hd + H + 1, window=window)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    rows = torch.arange(c.T, dtype=torch.int32, device=DEV)
    part_o = torch.empty(c.T * H * n_splits * hd, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(c.T * H * n_splits * 2, dtype=torch.float32, device=DEV)
    out = torch.full((c.T, H * hd), float("nan")).to(dtype).to(DEV)
    k.attn_row(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T, H,
               c.scale, window, n_splits, part_o, part_ml)
    want = c.reference()
    err = (out.double().cpu() - want).abs().max().item()
    assert err < _attn_tol(dtype), err


@pytest.mark.parametrize("case", [c for c in ATTN_CASES if c[2] in (32, 64, 128)] + [
    (8, 2, 32, 16, [700, 15, 16], [1, 1, 3], 0),
    (4, 4, 128, 16, [63, 64, 1000], [1, 2, 1], 100),
])
@pytest.mark.parametrize("n_splits,n_waves", [(1, 4), (3, 4), (8, 4), (1, 16), (1, 8), (2, 16), (1, 2)])
def test_attn_decode(case, n_splits, n_waves):
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(torch.bfloat16, H, Hkv, hd, ps, ctx, ql, seed=hd + H + 2, window=window)
    assert k.attn_decode_takes(torch.bfloat16, c.kv)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    rows = torch.arange(c.T, dtype=torch.int32, device=DEV)
    part_o = torch.empty(c.T * H * n_splits * hd, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(c.T * H * n_splits * 2, dtype=torch.float32, device=DEV)
    want = c.reference()
    for key_tile, here in ((32, 0), (64, 0), (32, 1), (64, 1), (32, 1), (32, 2), (64, 2)):
        # keys a wave takes at a time; the parts joined by a second kernel (0) or by the block that
        # arrives last (1; twice in a row: its counters are back at zero), short rows in fewer parts (2)
        out = torch.full((c.T, H * hd), float("nan")).to(torch.bfloat16).to(DEV)
        k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T, H,
                      c.scale, window, n_splits, part_o, part_ml, n_waves, key_tile=key_tile, join_in_kernel=here)
        err = (out.double().cpu() - want).abs().max().item()
        assert err < _attn_tol(torch.bfloat16), (key_tile, here, err)


@pytest.mark.parametrize("case", [c for c in ATTN_CASES if c[2] in (16, 32, 64)] + [
    (8, 2, 16, 16, [700, 15, 16], [1, 1, 3], 0),
    (3, 1, 64, 4, [63, 64, 1000], [1, 2, 1], 100),
    (25, 25, 64, 16, [511, 63, 1022, 64, 300], [1, 1, 1, 1, 1], 0),
])
@pytest.mark.parametrize("n_splits,n_waves", [(1, 4), (3, 4), (8, 2), (1, 16), (2, 8), (1, 1)])
def test_attn_decode_float32(case, n_splits, n_waves):
    """The same kernel over float caches: a key of 16, 32 or 64 floats in 4, 8 or 16 lanes."""
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(torch.float32, H, Hkv, hd, ps, ctx, ql, seed=hd + H + 3, window=window)
    assert k.attn_decode_takes(torch.float32, c.kv)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    rows = torch.arange(c.T, dtype=torch.int32, device=DEV)
    part_o = torch.empty(c.T * H * n_splits * hd, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(c.T * H * n_splits * 2, dtype=torch.float32, device=DEV)
    want = c.reference()
    for key_tile, here in ((32, 0), (64, 0), (32, 1), (64, 1), (32, 2)):
        out = torch.full((c.T, H * hd), float("nan"), dtype=torch.float32, device=DEV)
        k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T, H,
                      c.scale, window, n_splits, part_o, part_ml, n_waves, key_tile=key_tile, join_in_kernel=here)
        err = (out.double().cpu() - want).abs().max().item()
        assert err < _attn_tol(torch.float32), (key_tile, here, err)


def test_attn_decode_takes_keys_of_64_to_256_bytes():
    k = _k()
    for dtype, hd, ps, takes in [(torch.float32, 128, 16, False), (torch.float32, 48, 16, False),
                                 (torch.float32, 64, 2, False), (torch.float32, 64, 4, True),
                                 (torch.float32, 16, 16, True), (torch.bfloat16, 16, 16, False),
                                 (torch.bfloat16, 128, 4, True), (torch.bfloat16, 32, 8, False)]:
        c = PagedCase(dtype, 2, 2, hd, ps, [5], [1], seed=1)
        assert k.attn_decode_takes(dtype, c.kv) == takes, (dtype, hd, ps)
        if not takes:
            out = torch.empty(1, 2 * hd, dtype=dtype, device=DEV)
            rows = torch.zeros(1, dtype=torch.int32, device=DEV)
            with pytest.raises(RuntimeError, match="attn_decode"):
                k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, 1, 2,
                              c.scale)


@pytest.mark.parametrize("case", [
    (8, 2, 32, 16, [700, 15, 16, 0], [1, 1, 1, 1], 0),
    (25, 25, 64, 16, [511, 63, 1022, 64, 300], [1, 1, 1, 1, 1], 0),
    (4, 4, 128, 32, [63, 64, 1000], [1, 1, 1], 100),
])
@pytest.mark.parametrize("n_splits,n_waves", [(1, 2), (1, 16), (3, 4)])
def test_attn_decode_when_rows_are_requests(case, n_splits, n_waves):
    """A step in which every request brings one token: the kernel is told that item i is row i of
    request i and looks neither up (the row list it is handed here is garbage on purpose)."""
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(torch.bfloat16, H, Hkv, hd, ps, ctx, ql, seed=hd + H + 5, window=window)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    garbage = torch.full((c.T,), 10**6, dtype=torch.int32, device=DEV)
    part_o = torch.empty(c.T * H * n_splits * hd, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(c.T * H * n_splits * 2, dtype=torch.float32, device=DEV)
    outs = []
    for told in (True, False):
        out = torch.full((c.T, H * hd), float("nan")).to(torch.bfloat16).to(DEV)
        rows = garbage if told else torch.arange(c.T, dtype=torch.int32, device=DEV)
        k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, garbage if told else c.token_req, c.positions,
                      rows, c.T, H, c.scale, window, n_splits, part_o, part_ml, n_waves, rows_are_requests=told)
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    assert (outs[0].double().cpu() - c.reference()).abs().max().item() < _attn_tol(torch.bfloat16)


PREFILL_CASES = [c for c in ATTN_CASES if c[2] in (32, 64, 128)] + [
    (3, 3, 64, 16, [0, 100, 700], [300, 129, 5], 0),
    (4, 2, 32, 16, [5, 0], [260, 64], 0),
    (2, 1, 128, 32, [190, 0], [70, 200], 0),
    (5, 5, 64, 16, [0, 400], [333, 128], 90),
    (2, 2, 64, 48, [30, 0], [200, 150], 0),  # a page size that is no power of two
    (3, 1, 32, 80, [0, 77], [170, 40], 60),
]


@pytest.mark.parametrize("case", PREFILL_CASES)
def test_attn_prefill(case):
    k = _k()
    H, Hkv, hd, ps, ctx, ql, window = case
    c = PagedCase(torch.bfloat16, H, Hkv, hd, ps, ctx, ql, seed=hd + H + 3, window=window)
    assert k.attn_prefill_takes(torch.bfloat16, c.kv)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    tiles = c.tiles(k.attn_tile_sizes()[1])
    out = torch.full((c.T, H * hd), float("nan")).to(torch.bfloat16).to(DEV)
    k.attn_prefill(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, tiles,
                   tiles.shape[0], H, c.scale, window)
    err = (out.double().cpu() - c.reference()).abs().max().item()
    # the weights P are rounded to bfloat16 before they meet the values
    assert err < 2.5e-2, err


def test_attn_prefill_far_key_stands_out():
    """Every query of a long portion points at one far key of its own."""
    k = _k()
    H, hd, ps, n = 2, 64, 16, 320
    c = PagedCase(torch.bfloat16, H, H, hd, ps, [70], [n], seed=1)
    g = torch.Generator().manual_seed(2)
    far = [int(torch.randint(0, 70 + i + 1, (), generator=g)) for i in range(n)]
    for i in range(n):
        kf = c.k_full[0][far[i], 0].float()
        c.q[i, :hd] = (kf * (30.0 / (c.scale * float(kf.norm() ** 2)))).to(torch.bfloat16)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    tiles = c.tiles(k.attn_tile_sizes()[1])
    out = torch.empty(n, H * hd, dtype=torch.bfloat16, device=DEV)
    k.attn_prefill(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, tiles,
                   tiles.shape[0], H, c.scale, 0)
    got = out[:, :hd].double().cpu()
    want = torch.stack([c.v_full[0][f, 0] for f in far]).double()
    assert (got - want).abs().max().item() < 0.1
    assert (out.double().cpu() - c.reference()).abs().max().item() < 2.5e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_attn_decode_far_key_stands_out(dtype):
    """Keys streamed into registers: one key among hundreds carries the answer."""
    k = _k()
    H, hd, ps = 2, 64, 16
    for far in (0, 3, 4, 7, 8, 15, 16, 63, 64, 255, 256, 399, 400):
        c = PagedCase(dtype, H, H, hd, ps, [401], [1], seed=far)
        kf = c.k_full[0][far, 1].float()
        c.q[0, hd:] = (kf * (30.0 / (c.scale * float(kf.norm() ** 2)))).to(dtype)
        k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
        rows = torch.zeros(1, dtype=torch.int32, device=DEV)
        for n_splits, n_waves, key_tile in ((1, 4, 32), (4, 4, 32), (1, 16, 32), (1, 4, 64), (3, 8, 64)):
            out = torch.empty(1, H * hd, dtype=dtype, device=DEV)
            po = torch.empty(H * n_splits * hd, dtype=torch.float32, device=DEV)
            pm = torch.empty(H * n_splits * 2, dtype=torch.float32, device=DEV)
            k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, 1,
                          H, c.scale, 0, n_splits, po, pm, n_waves, key_tile=key_tile)
            v_far = c.v_full[0][far, 1].double()
            assert (out[0, hd:].double().cpu() - v_far).abs().max().item() < 0.1, (far, n_splits)
            assert (out.double().cpu() - c.reference()).abs().max().item() < _attn_tol(dtype)


def test_attn_far_key_stands_out():
    """One key among hundreds carries the answer: a dropped tile or page shows."""
    k = _k()
    H, hd, ps = 2, 32, 16
    for far in (0, 15, 16, 63, 64, 257, 400):
        c = PagedCase(torch.float32, H, H, hd, ps, [401], [1], seed=far)
        # the query points along key `far` of head 0 so that its score is 30:
        # that key takes nearly all the weight
        kf = c.k_full[0][far, 0].clone()
        c.q[0, :hd] = kf * (30.0 / (c.scale * float(kf.norm() ** 2)))
        k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
        rows = torch.zeros(1, dtype=torch.int32, device=DEV)
        want = c.reference()
        for n_splits in (1, 4):
            out = torch.empty(1, H * hd, dtype=torch.float32, device=DEV)
            po = torch.empty(H * n_splits * hd, dtype=torch.float32, device=DEV)
            pm = torch.empty(H * n_splits * 2, dtype=torch.float32, device=DEV)
            k.attn_row(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, 1,
                       H, c.scale, 0, n_splits, po, pm)
            assert (out.double().cpu() - want).abs().max().item() < 2e-5
            # and the answer is that key's value, to within the others' small weight
            v_far = c.v_full[0][far, 0].double()
            assert (out[0, :hd].double().cpu() - v_far).abs().max().item() < 0.1


def test_attn_refuses_bad_head_dim():
    k = _k()
    from mlx_lm_amd.ops.kernels import PagedKV

    pool = torch.zeros(4, 2, 1, 16, 24, device=DEV)
    kv = PagedKV(pool[:, 0], pool[:, 1])
    q = torch.zeros(1, 24, device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        k.attn_row(q.clone(), q, kv, bt, z, z, z, 1, 1, 1.0)


# ---------------------------------------------------------------------------
# sampling


def _sample(logits, temp=0.0, top_p=0.0, min_p=0.0, min_keep=1, top_k=0, xtc_prob=0.0, xtc_thr=0.1,
            seed=0, counter=0, special=None, want_logprobs=False):
    k = _k()
    n, V = logits.shape

    def col(v, dt):
        if isinstance(v, (list, tuple)):
            return torch.tensor(v, dtype=dt, device=DEV)
        return torch.full((n,), v, dtype=dt, device=DEV)

    tokens = torch.empty(n, dtype=torch.int32, device=DEV)
    tlp = torch.empty(n, dtype=torch.float32, device=DEV)
    lp = torch.empty(n, V, dtype=torch.float32, device=DEV) if want_logprobs else None
    sp = torch.tensor(special, dtype=torch.int32, device=DEV) if special else None
    k.sample_rows(tokens, tlp, logits, col(temp, torch.float32), col(top_p, torch.float32),
                  col(min_p, torch.float32), col(min_keep, torch.int32), col(top_k, torch.int32),
                  col(xtc_prob, torch.float32), col(xtc_thr, torch.float32), col(seed, torch.int64),
                  col(counter, torch.int32), sp, lp)
    return tokens.cpu(), tlp.cpu(), (lp.cpu() if lp is not None else None)


def test_sample_greedy_and_logprobs():
    logits = _rand((9, 1000), torch.float32, 20, 3.0)
    logits[3, 17] = logits[3, 500] = 50.0  # a tie goes to the lower index
    tok, tlp, lp = _sample(logits, want_logprobs=True)
    want_lp = plain.log_softmax(logits.double().cpu())
    assert torch.equal(tok.long(), want_lp.argmax(-1))
    assert tok[3] == 17
    assert torch.allclose(lp.double(), want_lp, atol=1e-5)
    assert torch.allclose(tlp.double(), want_lp.gather(1, tok.long()[:, None])[:, 0], atol=1e-5)


def _support(probs_row, n=4000, **kw):
    """Empirical distribution of n draws (n rows, one counter each)."""
    V = probs_row.numel()
    logits = torch.log(probs_row).float().to(DEV)[None].repeat(n, 1).contiguous()
    tok, _, _ = _sample(logits, counter=list(range(n)), **kw)
    return torch.bincount(tok.long(), minlength=V).double() / n


def test_sample_temperature_distribution():
    p = torch.tensor([0.5, 0.25, 0.125, 0.0625, 0.0625])
    freq = _support(p, n=8000, temp=1.0, seed=5)
    assert (freq - p.double()).abs().max() < 0.02
    # temperature 0.5 squares the probabilities
    q = p.double() ** 2
    q = q / q.sum()
    freq = _support(p, n=8000, temp=0.5, seed=6)
    assert (freq - q).abs().max() < 0.02


def test_sample_filters_match_reference_vectors():
    # vectors of the reference's tests/test_sample_utils.py:19-105
    p = torch.tensor([0.9, 1e-9, 1e-9, 0.1])
    f = _support(p / p.sum(), n=500, temp=1.0, top_p=0.3, seed=1)
    assert f[0] == 1.0
    p = torch.tensor([1e-9, 0.5, 0.4, 0.1])
    f = _support(p / p.sum(), n=6000, temp=1.0, top_p=0.6, seed=2)
    assert f[0] == 0 and f[3] == 0 and abs(f[1] - 0.5556) < 0.03
    f = _support(p / p.sum(), n=6000, temp=1.0, top_p=0.95, seed=3)
    assert f[0] == 0 and abs(f[1] - 0.5) < 0.03 and abs(f[3] - 0.1) < 0.02
    p = torch.tensor([0.6, 1e-9, 0.1, 0.3])
    f = _support(p / p.sum(), n=6000, temp=1.0, top_k=2, seed=4)
    assert f[1] == 0 and f[2] == 0 and abs(f[0] - 0.6667) < 0.03
    p = torch.tensor([0.9, 1e-9, 1e-9, 0.1])
    f = _support(p / p.sum(), n=500, temp=1.0, min_p=0.8, seed=5)
    assert f[0] == 1.0
    f = _support(p / p.sum(), n=4000, temp=1.0, min_p=0.05, seed=6)
    assert abs(f[0] - 0.9) < 0.03 and f[1] == 0
    # min_tokens_to_keep keeps the two best although min_p would drop one
    f = _support(p / p.sum(), n=4000, temp=1.0, min_p=0.8, min_keep=2, seed=7)
    assert abs(f[3] - 0.1) < 0.03 and f[1] == 0 and f[2] == 0


def test_sample_filters_against_plain_on_random_rows():
    g = torch.Generator().manual_seed(9)
    V = 777
    logits = (torch.randn(6, V, generator=g) * 2.5).float()
    lp = plain.log_softmax(logits.double())
    for kw, filt in [
        (dict(top_p=0.7), lambda x: plain.top_p_filter(x, 0.7)),
        (dict(top_k=13), lambda x: plain.top_k_filter(x, 13)),
        (dict(min_p=0.2, min_keep=5), lambda x: plain.min_p_filter(x, 0.2, 5)),
        (dict(top_p=0.9, min_p=0.05, top_k=20),
         lambda x: plain.top_k_filter(plain.min_p_filter(plain.top_p_filter(x, 0.9), 0.05), 20)),
        (dict(xtc_prob=1.0, xtc_thr=0.02, special=[int(lp[0].argmax())]),
         lambda x: plain.xtc_filter(x, 0.02, [int(lp[0].argmax())])),
    ]:
        allowed = torch.isfinite(filt(lp.clone()))
        seen = torch.zeros_like(allowed)
        for counter in range(60):
            tok, _, _ = _sample(logits.to(DEV), temp=1.5, seed=11, counter=counter, **kw)
            seen[torch.arange(6), tok.long()] = True
        assert not (seen & ~allowed).any(), kw
        # small supports are covered completely
        small = allowed.sum(-1) <= 6
        assert torch.equal((seen & allowed)[small], allowed[small]), kw


@pytest.mark.parametrize("shape", ["peaked", "flat"])
def test_sample_filters_at_large_vocabularies(shape):
    """The filters' thresholds at vocabularies beyond the kernel's list of candidates: a peaked row
    (the thresholds come from the list) and a flat one (no list: passes over the row).  A high
    temperature makes the draw nearly uniform over what is kept, so the kept set shows."""
    g = torch.Generator().manual_seed(3)
    if shape == "peaked":
        V, n = 50257, 1200
        logits = -0.35 * torch.arange(V).double() ** 0.75 + 0.3 * torch.randn(V, generator=g).double()
        logits = logits[torch.randperm(V, generator=g)]
        cases = [dict(top_p=0.8), dict(top_k=13), dict(min_p=0.3, min_keep=9), dict(top_p=0.95, top_k=25)]
    else:
        V, n = 20000, 1200
        logits = 0.01 * torch.randn(V, generator=g).double()
        cases = [dict(top_p=0.00045), dict(top_k=7), dict(min_p=0.999, min_keep=6), dict(top_p=0.002, top_k=11)]
    lp = plain.log_softmax(logits.float().double()[None])[0]
    probs = lp.exp()
    for kw in cases:
        x = lp.clone()[None]
        if "top_p" in kw:
            x = plain.top_p_filter(x, kw["top_p"])
        if "min_p" in kw:
            x = plain.min_p_filter(x, kw["min_p"], kw.get("min_keep", 1))
        if "top_k" in kw:
            x = plain.top_k_filter(x, kw["top_k"])
        allowed = torch.isfinite(x[0])
        assert 1 <= int(allowed.sum()) <= 60, (kw, int(allowed.sum()))
        rows = logits.float().to(DEV)[None].repeat(n, 1).contiguous()
        tok, _, _ = _sample(rows, temp=200.0, seed=21, counter=list(range(n)), **kw)
        seen = torch.bincount(tok.long(), minlength=V) > 0
        assert torch.equal(seen, allowed), (shape, kw, int(seen.sum()), int(allowed.sum()))


def test_sample_seed_and_batch_independence():
    logits = _rand((5, 300), torch.float32, 30, 2.0)
    a, _, _ = _sample(logits, temp=0.9, seed=[1, 2, 3, 4, 5], counter=[0, 1, 2, 3, 4])
    b, _, _ = _sample(logits, temp=0.9, seed=[1, 2, 3, 4, 5], counter=[0, 1, 2, 3, 4])
    assert torch.equal(a, b)
    # row 2 alone gives the same token as row 2 in the batch
    c, _, _ = _sample(logits[2:3].contiguous(), temp=0.9, seed=[3], counter=[2])
    assert c[0] == a[2]
    draws = {int(_sample(logits[:1].contiguous(), temp=2.0, seed=[7], counter=[i])[0][0]) for i in range(16)}
    assert len(draws) > 1


def test_logit_bias_and_penalties():
    k = _k()
    V = 50
    logits = _rand((3, V), torch.float32, 40)
    base = logits.double().cpu()
    offsets = torch.tensor([0, 2, 2, 5], dtype=torch.int32, device=DEV)
    idx = torch.tensor([0, 7, 3, 3, 9], dtype=torch.int32, device=DEV)
    val = torch.tensor([2000.0, -1.0, 0.5, 0.25, 4.0], device=DEV)
    x = logits.clone()
    k.apply_logit_bias(x, offsets, idx, val)
    want = base.clone()
    want[0, 0] += 2000
    want[0, 7] -= 1
    want[2, 3] += 0.75
    want[2, 9] += 4
    assert torch.allclose(x.double().cpu(), want, atol=1e-4)

    hist_rows = [[5, 6, 5, 7, 5], [], [1, 2, 3, 4, 1, 1, 9]]
    hist = torch.tensor(sum(hist_rows, []), dtype=torch.int32, device=DEV)
    offsets = torch.tensor([0, 5, 5, 12], dtype=torch.int32, device=DEV)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    rep, pres, freq = [1.3, 1.3, 0.0], [0.5, 0.0, 0.25], [0.0, 0.1, 0.2]
    rep_ctx, pres_ctx, freq_ctx = [20, 20, 20], [2, 20, 3], [20, 20, 4]
    x = logits.clone()
    k.apply_penalties(x, offsets, hist, f32(rep), i32(rep_ctx), f32(pres), i32(pres_ctx), f32(freq),
                      i32(freq_ctx))
    for r in range(3):
        want = base[r].clone()
        if rep[r]:
            want = plain.repetition_penalty(want, hist_rows[r], rep[r], rep_ctx[r])
        if pres[r]:
            want = plain.presence_penalty(want, hist_rows[r], pres[r], pres_ctx[r])
        if freq[r]:
            want = plain.frequency_penalty(want, hist_rows[r], freq[r], freq_ctx[r])
        assert torch.allclose(x[r].double().cpu(), want, atol=1e-5), r


# ---------------------------------------------------------------------------
# the decode projection: norm fused in front, cache scatter fused behind


@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (7, 1000, 96), (16, 80, 200), (8, 4800, 1600),
                                   (9, 1600, 6400), (13, 333, 1608), (16, 257, 3200)])
@pytest.mark.parametrize("mode", ["plain", "gelu", "accumulate", "f32out"])
@pytest.mark.parametrize("normed", [False, True])
@pytest.mark.parametrize("packed", [False, True])
def test_gemm_bf16_decode(M, N, K, mode, normed, packed):
    k = _k()
    from mlx_lm_amd.ops import build

    lib = build.load("gemm_bf16_decode")
    if not lib.gemm_bf16_decode_takes(M, K, int(normed), 1):
        assert K > 2048 and normed  # the only sizes of this list it leaves to the general kernels
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    if normed:
        x = _rand((M, K), torch.float32, 10, 2.0) + 0.3
        gamma, beta = 1 + _rand((K,), torch.float32, 14, 0.1), _rand((K,), torch.float32, 15, 0.1)
        a = k.NormedInput(lambda shape, dtype: torch.empty(shape, dtype=dtype, device=DEV), x, gamma, beta,
                          1e-5, torch.bfloat16)
        a_ref = plain.layer_norm(x.double().cpu(), gamma.double().cpu(), beta.double().cpu(), 1e-5)
        a_ref = a_ref.to(torch.bfloat16).double()  # the kernel rounds the normed rows to bfloat16 too
    else:
        a = _rand((M, K), torch.bfloat16, 10)
        a_ref = a.double().cpu()
    ref = plain.linear(a_ref, w.double().cpu(), bias.double().cpu())
    if packed:
        w = k.PackedWeight(w)  # tiles in the lanes' order, with a row-major copy beside
    slack = 3e-2 * math.sqrt(K) * 0.1 if normed else 0.0  # a normed value may round the other way
    if mode == "accumulate":
        out = _rand((M, N), torch.float32, 13)
        want = out.double().cpu() + ref
        k.linear(out, a, w, bias, accumulate=True)
        tol = 1e-4 * math.sqrt(K) + slack
    elif mode == "f32out":
        out = torch.empty(M, N, dtype=torch.float32, device=DEV)
        k.linear(out, a, w, bias)
        want, tol = ref, 1e-4 * math.sqrt(K) + slack
    else:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        k.linear(out, a, w, bias, gelu=(mode == "gelu"))
        want = plain.gelu_tanh(ref) if mode == "gelu" else ref
        tol = None
    got = out.double().cpu()
    if tol is None:
        assert torch.allclose(got, want, rtol=2**-7, atol=1e-3 + slack), (got - want).abs().max()
    else:
        assert (got - want).abs().max().item() < tol, (got - want).abs().max()


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + [(2048, 1600, 1600), (260, 200, 6400)])
def test_gemm_bf16_reads_weights_kept_in_packed_order_only(M, N, K):
    """Every kernel of the many-row products (all tile shapes, the skinny kernel, the splits of K)
    reads weights that exist in the decode kernels' packed order only: bit for bit what the same
    kernel makes of the row-major matrix, at sizes with ragged edges (features that are no
    multiple of 16, K no multiple of 64 or shorter than a k-block)."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    packed = k.PackedWeight(w.clone(), keep_rows=False)
    assert packed.w is None and not packed.c.w
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    variants = [(v, None) for v in ((1, 2, 3, 4, 5, 6, 7) if M <= 64 else (1, 3, 4, 5, 6, 7))]
    if M > 16 and K >= 192:
        variants += [(1, 3), (5, 2), (6, 3), (0, 2)]  # K in parts
    variants.append((0, None))  # the library's own choice
    for variant, splits in variants:
        outs = []
        for weights in (w, packed):
            out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
            k.linear(out, a, weights, bias, gelu=True, variant=variant, splits=splits)
            outs.append(out)
        # (left to itself the library takes another kernel for 17 to 64 rows of packed weights,
        # which adds in another order)
        if variant != 0 or not 16 < M <= 64:
            assert torch.equal(outs[0], outs[1]), (variant, splits)
        assert torch.allclose(outs[1].double().cpu(), plain.gelu_tanh(ref), rtol=2**-7, atol=1e-3), (variant, splits)


@pytest.mark.parametrize("M,N,K", [(17, 48, 64), (33, 257, 384), (64, 4800, 1600), (40, 1600, 6400), (64, 333, 1608),
                                   (48, 80, 200), (20, 100, 520), (32, 4800, 1600), (24, 1600, 6400), (30, 333, 1608)])
@pytest.mark.parametrize("mode", ["plain", "gelu", "accumulate", "f32out"])
@pytest.mark.parametrize("packed", [False, True])
def test_gemm_bf16_17_to_64_rows(M, N, K, mode, packed):
    """17 to 64 rows, the library's own choice of kernel and parts: with packed weights the kernel
    that holds a block's weights in registers (32 features a block; K in parts where that gives
    few blocks or a part would be longer than a block holds; from 49 rows on two groups of rows,
    a block each), otherwise tiles of 32 x 128 and 64 x 128 with K split over blocks."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    if packed:
        w = k.PackedWeight(w)
    if mode == "accumulate":
        out = _rand((M, N), torch.float32, 13)
        want = out.double().cpu() + ref
        k.linear(out, a, w, bias, accumulate=True)
        tol = 1e-4 * math.sqrt(K)
    elif mode == "f32out":
        out = torch.empty(M, N, dtype=torch.float32, device=DEV)
        k.linear(out, a, w, bias)
        want, tol = ref, 1e-4 * math.sqrt(K)
    else:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        k.linear(out, a, w, bias, gelu=(mode == "gelu"))
        want, tol = (plain.gelu_tanh(ref) if mode == "gelu" else ref), None
    got = out.double().cpu()
    if tol is None:
        assert torch.allclose(got, want, rtol=2**-7, atol=1e-3), (got - want).abs().max()
    else:
        assert (got - want).abs().max().item() < tol, (got - want).abs().max()


@pytest.mark.parametrize("M,N,K", [(17, 48, 1024), (48, 1600, 6400), (24, 333, 1608), (33, 4800, 1600), (32, 1000, 1792),
                                   (41, 72, 136), (20, 100, 1856)])
def test_gemm_bf16_rows_kernel_in_parts_and_with_the_cache_scatter(M, N, K):
    """The kernel for 17 to 64 rows, asked for directly: whole and with K in 2, 3 and 8 parts (the
    same bits run after run), at the longest slice it holds (28 k-blocks), refusing a longer one,
    and with keys and values going to their pages from its epilogue or from the second kernel."""
    k = _k()
    from mlx_lm_amd.ops import build

    lib = build.load("gemm_bf16_decode")
    n_blocks = (K + 63) // 64
    assert lib.gemm_bf16_rows_takes(M, K, 1) == (1 if n_blocks <= 28 else 0)
    assert lib.gemm_bf16_rows_takes(16, K, 1) == 0 and lib.gemm_bf16_rows_takes(65, K, 1) == 0
    auto = lib.gemm_bf16_rows_splits(M, N, K, 0)
    assert auto >= 1 and (n_blocks + auto - 1) // auto <= 28
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    packed = k.PackedWeight(w, keep_rows=False)
    for splits in (None, 2, 3, 8):
        if splits is not None and (splits > n_blocks or (n_blocks + splits - 1) // splits > 28):
            continue
        if splits is None and n_blocks > 28:
            continue
        outs = []
        for _ in range(2):
            out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
            k.linear(out, a, packed, bias, gelu=True, splits=splits or 1)
            outs.append(out)
        assert torch.equal(outs[0], outs[1]), splits
        assert torch.allclose(outs[0].double().cpu(), plain.gelu_tanh(ref), rtol=2**-7, atol=1e-3), splits
    # the cache scatter: rows of several requests, grouped key heads, a head size that is no power of two
    for H, Hkv, hd, M_per in ((5, 5, 64, [20, 1, 10]), (4, 2, 80, [17, 30])):
        ps, D = 16, 264
        c = PagedCase(torch.bfloat16, H, Hkv, hd, ps, [7 + 20 * i for i in range(len(M_per))], M_per, seed=M)
        rows, qw, kw = sum(M_per), H * hd, Hkv * hd
        w2 = _rand((qw + 2 * kw, D), torch.bfloat16, 3, 0.2)
        b2 = _rand((qw + 2 * kw,), torch.float32, 4, 0.1)
        a2 = _rand((rows, D), torch.bfloat16, 5)
        c.pool.fill_(float("nan"))
        plain_out = torch.empty(rows, qw + 2 * kw, dtype=torch.bfloat16, device=DEV)
        k.linear(plain_out, a2, k.PackedWeight(w2, keep_rows=False), b2, splits=1)
        want = plain.linear(a2.double().cpu(), w2.double().cpu(), b2.double().cpu())
        assert torch.allclose(plain_out.double().cpu(), want, rtol=2**-7, atol=1e-3)
        k.kv_write(plain_out[:, qw : qw + kw], plain_out[:, qw + kw :], c.kv, c.block_table_dev, c.token_req, c.positions)
        want_pool = c.pool.clone()
        written = ~torch.isnan(want_pool.float())
        for splits in (1, 2):
            c.pool.fill_(float("nan"))
            out = torch.full((rows, qw + 2 * kw), float("nan"), dtype=torch.bfloat16, device=DEV)
            sc = k.KVScatter(c.kv, c.block_table_dev, c.token_req, c.positions, qw)
            k.linear(out, a2, k.PackedWeight(w2, keep_rows=False), b2, scatter=sc, splits=splits)
            if splits == 1:  # (parts are added in another order than one walk through K)
                assert torch.equal(out[:, :qw], plain_out[:, :qw])
                assert torch.equal(c.pool[written], want_pool[written])
            else:
                assert torch.allclose(out[:, :qw].float(), plain_out[:, :qw].float(), rtol=2**-6, atol=2e-3)
                assert torch.allclose(c.pool[written].float(), want_pool[written].float(), rtol=2**-6, atol=2e-3)
            assert torch.isnan(out[:, qw:].float()).all()
            assert written.any() and torch.isnan(c.pool[~written].float()).all()


@pytest.mark.parametrize("M,N,K", [(17, 48, 64), (33, 257, 1536), (64, 4800, 1600), (40, 1600, 6400), (49, 333, 1608),
                                   (48, 80, 1600), (20, 100, 520), (32, 4800, 1600), (63, 1600, 1792), (50, 6400, 1600)])
def test_rows_in_the_packed_order_into_and_out_of_the_product_of_17_to_64_rows(M, N, K):
    """The product of 17 to 64 rows takes its rows row-major or in tiles of 16 rows x 64 columns laid
    out like the packed weights' tiles, and writes a bfloat16 result in that order where asked: the
    same bits either way, whole and with K in parts (the second kernel then writes the order), and
    whatever lies in the tiles beyond the last row and column (NaN here)."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = k.PackedWeight(_rand((N, K), torch.bfloat16, 11, 0.1), keep_rows=False)
    bias = _rand((N,), torch.float32, 12)
    # (beyond 32 rows that kernel takes a product only where K is long: 1,536 columns or more)
    assert k.wants_packed_rows(w, M) and not k.wants_packed_rows(w, 16) and not k.wants_packed_rows(w, 65)
    assert k.wants_packed_rows(w, 33) == (K >= 1536)
    pa = k.PackedRows.of(a)
    assert torch.equal(pa.rows(), a)
    # what the tiles hold beyond the matrix must not matter
    Mp, Kp = (M + 15) // 16 * 16, (K + 63) // 64 * 64
    junk = torch.full((Mp, Kp), float("nan"), dtype=torch.bfloat16, device=DEV)
    junk[:M, :K] = a
    pa = k.PackedRows(k.PackedRows.of(junk).data, (M, K))
    n_blocks = (K + 63) // 64
    for splits in (None, 2, 3):
        if splits is not None and (splits > n_blocks or (n_blocks + splits - 1) // splits > 28):
            continue
        for gelu in (False, True):
            want = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            k.linear(want, a, w, bias, gelu=gelu, splits=splits)
            got = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            k.linear(got, pa, w, bias, gelu=gelu, splits=splits)
            assert torch.equal(got, want), (splits, gelu)
            out = k.PackedRows.empty(M, N, DEV)
            out.data.fill_(float("nan"))
            k.linear(out, pa, w, bias, gelu=gelu, splits=splits)
            assert torch.equal(out.rows(), want), (splits, gelu)
        h = _rand((M, N), torch.float32, 13)
        h2 = h.clone()
        k.linear(h, a, w, bias, accumulate=True, splits=splits)
        k.linear(h2, pa, w, bias, accumulate=True, splits=splits)
        assert torch.equal(h, h2), splits
    ref = plain.linear(a.double().cpu(), w_rows(w, N, K).double().cpu(), bias.double().cpu())
    assert torch.allclose(want.double().cpu(), plain.gelu_tanh(ref), rtol=2**-7, atol=1e-3)
    # elsewhere the order is refused, not misread
    few = k.PackedRows.of(a[:8].contiguous())
    with pytest.raises(RuntimeError, match="packed order"):
        k.linear(torch.empty(8, N, dtype=torch.bfloat16, device=DEV), few, w, bias)


def w_rows(w, N, K):
    """A ``PackedWeight``'s matrix back in rows."""
    k = _k()
    return k.PackedRows(w.packed, (N, K)).rows()


def test_the_sum_and_norm_and_decode_attention_write_the_packed_order():
    k = _k()
    M, N, K = 40, 1600, 1792
    a = _rand((M, K), torch.bfloat16, 1)
    w = k.PackedWeight(_rand((N, K), torch.bfloat16, 2, 0.1), keep_rows=False)
    bias, gamma, beta = _rand((N,), torch.float32, 3), 1 + _rand((N,), torch.float32, 4, 0.1), _rand((N,), torch.float32, 5, 0.1)
    h0 = _rand((M, N), torch.float32, 6)
    outs = []
    for packed in (False, True):
        h = h0.clone()
        pending = k.PendingSum()
        pending.allowed = True
        k.linear(h, a, w, bias, accumulate=True, splits=4, pending=pending)
        assert pending.waits_on(h) and pending.can_norm(h)
        y = k.PackedRows.empty(M, N, DEV) if packed else torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        pending.settle_normed(y, gamma, beta, 1e-5)
        outs.append((h, y.rows() if packed else y))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    want = plain.layer_norm(outs[0][0].double().cpu(), gamma.double().cpu(), beta.double().cpu(), 1e-5)
    assert torch.allclose(outs[0][1].double().cpu(), want, atol=2e-2, rtol=2e-2)
    # decode attention: 37 rows of 5 heads of 64, each a request of its own
    H, hd, n = 5, 64, 37
    c = PagedCase(torch.bfloat16, H, H, hd, 16, [3 + 11 * i for i in range(n)], [1] * n, seed=8)
    k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
    rows = torch.arange(c.T, dtype=torch.int32, device=DEV)
    plain_out = torch.empty(c.T, H * hd, dtype=torch.bfloat16, device=DEV)
    k.attn_decode(plain_out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T, H, c.scale)
    for n_splits in (1, 3):
        packed_out = k.PackedRows.empty(c.T, H * hd, DEV)
        part_o = torch.empty(c.T * H * n_splits * hd, device=DEV)
        part_ml = torch.empty(c.T * H * n_splits * 2, device=DEV)
        k.attn_decode(packed_out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T, H, c.scale,
                      n_splits=n_splits, part_o=part_o, part_ml=part_ml)
        if n_splits == 1:
            assert torch.equal(packed_out.rows(), plain_out)
        else:
            assert torch.allclose(packed_out.rows().float(), plain_out.float(), rtol=2**-6, atol=2e-3)
    assert torch.allclose(plain_out.double().cpu(), c.reference(), rtol=2**-6, atol=3e-3)


@pytest.mark.parametrize("M,N,K", [(1, 48, 1024), (8, 1600, 6400), (16, 80, 200), (16, 1600, 6400), (11, 333, 1608),
                                   (17, 48, 1024), (64, 1600, 6400), (40, 333, 1608), (33, 4800, 1600),
                                   (65, 257, 1608), (130, 300, 200), (300, 1600, 1600), (72, 96, 128)])
@pytest.mark.parametrize("mode", ["plain", "accumulate", "gelu"])
def test_gemm_bf16_decode_split_k(M, N, K, mode):
    """K split over blocks (the decode kernels up to 16 rows, the tile kernels beyond): partial sums
    in the workspace, added in the order of the splits by a second kernel, so a number of splits
    gives the same bits run after run."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    for splits in (2, 3, 8):
        if splits > (K + 63) // 64:
            continue
        outs = []
        for _ in range(3):
            if mode == "accumulate":
                out = _rand((M, N), torch.float32, 13)
                k.linear(out, a, w, bias, accumulate=True, splits=splits)
                want = _rand((M, N), torch.float32, 13).double().cpu() + ref
                tol = 1e-4 * math.sqrt(K)
            elif mode == "gelu":
                out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
                k.linear(out, a, w, bias, gelu=True, splits=splits)
                want = plain.gelu_tanh(ref)
                tol = 2**-7 * float(want.abs().max()) + 1e-3
            else:
                out = torch.empty(M, N, dtype=torch.float32, device=DEV)
                k.linear(out, a, w, bias, splits=splits)
                want, tol = ref, 1e-4 * math.sqrt(K)
            outs.append(out.clone())
        assert (outs[0].double().cpu() - want).abs().max().item() < tol, splits
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), splits


@pytest.mark.parametrize("M,N,K", [(33, 257, 1608), (64, 1600, 1600), (50, 96, 128), (40, 333, 200)])
@pytest.mark.parametrize("mode", ["plain", "accumulate", "gelu"])
def test_gemm_bf16_small_tiles_split_k(M, N, K, mode):
    """33 to 64 rows: tiles of 64 x 128 with K split over blocks, summed by the second kernel."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 20)
    w = _rand((N, K), torch.bfloat16, 21, 0.1)
    bias = _rand((N,), torch.float32, 22)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    for splits in (1, 2, 5):
        if splits > (K + 63) // 64:
            continue
        if mode == "accumulate":
            out = _rand((M, N), torch.float32, 23)
            k.linear(out, a, w, bias, accumulate=True, variant=5, splits=splits)
            want, tol = _rand((M, N), torch.float32, 23).double().cpu() + ref, 1e-4 * math.sqrt(K)
        elif mode == "gelu":
            out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            k.linear(out, a, w, bias, gelu=True, variant=5, splits=splits)
            want = plain.gelu_tanh(ref)
            tol = 2**-7 * float(want.abs().max()) + 1e-3
        else:
            out = torch.empty(M, N, dtype=torch.float32, device=DEV)
            k.linear(out, a, w, bias, variant=5, splits=splits)
            want, tol = ref, 1e-4 * math.sqrt(K)
        assert (out.double().cpu() - want).abs().max().item() < tol, splits


@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (8, 1600, 6400), (16, 96, 384), (40, 240, 200), (64, 1600, 1600),
                                   (5, 4100, 512), (100, 1600, 1600), (200, 240, 456)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_pending_sum_is_added_by_the_norm(M, N, K, out_dtype):
    """A split projection into the residual stream may stop at its partial sums; the norm that reads the
    stream next adds them, writes the stream and norms the new rows in one kernel.  A bias of 3 on one
    feature and a stream row far from zero show a sum or a shift left out."""
    k = _k()
    a = _rand((M, K), torch.bfloat16, 10)
    w = _rand((N, K), torch.bfloat16, 11, 0.1)
    bias = _rand((N,), torch.float32, 12)
    bias[N // 3] = 3.0
    h0 = _rand((M, N), torch.float32, 13)
    h0[M // 2] += 5.0
    gamma = 1 + _rand((N,), torch.float32, 5, 0.1)
    beta = _rand((N,), torch.float32, 6, 0.1)
    eps = 1e-5
    want_h = h0.double().cpu() + plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    want_y = plain.layer_norm(want_h, gamma.double().cpu(), beta.double().cpu(), eps)
    tol_y = 2e-2 if out_dtype == torch.bfloat16 else 1e-4 * math.sqrt(K)
    for splits in (2, 4):
        if splits > (K + 63) // 64:
            continue
        # fused: sum, stream and norm in one kernel
        h = h0.clone()
        pending = k.PendingSum()
        pending.allowed = True
        k.linear(h, a, w, bias, accumulate=True, splits=splits, pending=pending)
        assert pending.waits_on(h) and torch.equal(h, h0)  # nothing added yet
        assert pending.can_norm(h) == (N % 4 == 0 and N <= 8192)
        y = torch.empty(M, N, dtype=out_dtype, device=DEV)
        if pending.can_norm(h):
            pending.settle_normed(y, gamma, beta, eps)
        else:
            pending.settle()
            k.layernorm(y, h, gamma, beta, eps)
        assert not pending.waits_on(h)
        assert (h.double().cpu() - want_h).abs().max().item() < 1e-4 * math.sqrt(K)
        assert torch.allclose(y.double().cpu(), want_y, atol=tol_y, rtol=tol_y)
        # plain settle gives the same stream as the product that adds at once
        h2 = h0.clone()
        pending.allowed = True
        k.linear(h2, a, w, bias, accumulate=True, splits=splits, pending=pending)
        pending.settle()
        h3 = h0.clone()
        k.linear(h3, a, w, bias, accumulate=True, splits=splits)
        assert torch.equal(h2, h3)
        assert (h2.double().cpu() - want_h).abs().max().item() < 1e-4 * math.sqrt(K)
        # not allowed: the product finishes by itself
        pending.allowed = False
        h4 = h0.clone()
        k.linear(h4, a, w, bias, accumulate=True, splits=splits, pending=pending)
        assert not pending.waits_on(h4) and torch.equal(h4, h3)


def test_reading_weights_ahead_changes_nothing():
    """The blocks that read the next product's weights ahead (in the fused sum-and-norm and in decode
    attention) only read: results are what they are without them, for weights whose last chunk is
    short of nothing (padded) and counts of chunks that are no multiple of eight."""
    k = _k()
    for n_feat, K in ((2400 + 16 * 3, 192), (16 * 151, 64)):
        w = k.for_decode(_rand((n_feat, K), torch.bfloat16, 3, 0.1))
        assert k.read_ahead_pays(w, 8) and w.n_chunks * w.chunk_bytes == w.packed.numel() * 2
        assert not k.read_ahead_pays(k.for_decode(_rand((1600, 64), torch.bfloat16, 3)), 8)  # 8 features a block
        assert not k.read_ahead_pays(w, 17)
        # the fused sum-and-norm
        M, N = 8, 96
        ws = _rand((3, M, N), torch.float32, 4)
        bias, gamma, beta = _rand((N,), torch.float32, 5), 1 + _rand((N,), torch.float32, 6, 0.1), _rand((N,), torch.float32, 7)
        h0 = _rand((M, N), torch.float32, 8)
        outs = []
        for ahead in (None, w):
            h, y = h0.clone(), torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            k.sum_partials_norm(h, ws, 3, bias, gamma, beta, 1e-5, y, ahead=ahead)
            outs.append((h, y))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
        # decode attention: one row and eight, with and without split keys
        for ctx, n_splits in (([300], 1), ([40, 7, 90, 3, 200, 64, 65, 1], 1), ([500, 20], 2)):
            H, hd = 3, 64
            c = PagedCase(torch.bfloat16, H, H, hd, 16, ctx, [1] * len(ctx), seed=len(ctx))
            k.kv_write(c.k_new.to(DEV), c.v_new.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions)
            rows = torch.arange(c.T, dtype=torch.int32, device=DEV)
            po = torch.empty(c.T * H * n_splits * hd, dtype=torch.float32, device=DEV)
            pm = torch.empty(c.T * H * n_splits * 2, dtype=torch.float32, device=DEV)
            res = []
            for ahead in (None, w):
                out = torch.full((c.T, H * hd), float("nan")).to(torch.bfloat16).to(DEV)
                k.attn_decode(out, c.q.to(DEV), c.kv, c.block_table_dev, c.token_req, c.positions, rows, c.T,
                              H, c.scale, 0, n_splits, po, pm, 4, ahead=ahead, ahead_chunks=10**6)
                res.append(out)
            assert torch.equal(res[0], res[1])
            assert (res[1].double().cpu() - c.reference()).abs().max().item() < _attn_tol(torch.bfloat16)


def test_default_splits_fill_the_gpu():
    """The library's own choice: no split where feature blocks alone fill the GPU, some where they do not."""
    k = _k()
    lib = k.build.load("gemm_bf16_decode")
    assert lib.gemm_bf16_decode_splits(8, 4800, 1600, 0, 0) == 1
    assert lib.gemm_bf16_decode_splits(8, 1600, 6400, 0, 0) > 1
    assert lib.gemm_bf16_decode_splits(1, 1600, 6400, 0, 0) == 1  # a row or two: the norm prologue is cheaper
    assert lib.gemm_bf16_decode_splits(8, 1600, 1600, 1, 0) == 1  # the norm prologue needs whole rows
    assert lib.gemm_bf16_decode_splits(16, 1600, 6400, 0, 0) > 1
    assert lib.gemm_bf16_decode_splits(16, 50257, 1600, 0, 0) == 1
    assert lib.gemm_bf16_decode_splits(17, 1600, 6400, 0, 0) == 1  # (not this library's rows)
    assert lib.gemm_bf16_decode_splits(8, 64, 64, 0, 0) == 1
    assert lib.gemm_bf16_decode_splits(8, 64, 64, 0, 2) == 1  # one k-block cannot be split
    assert lib.gemm_bf16_decode_splits(8, 64, 200, 0, 2) == 2
    tiles = k.build.load("gemm_bf16")
    # (rows, features, K, the sum is left to the next norm, forced parts)
    assert tiles.gemm_bf16_splits(16, 1600, 6400, 1, 0) == 1  # (the decode kernels' rows)
    assert tiles.gemm_bf16_splits(17, 1600, 6400, 1, 0) > 8
    assert tiles.gemm_bf16_splits(64, 50257, 1600, 0, 0) == 1  # (many tiles fill the GPU as they are)
    assert tiles.gemm_bf16_splits(64, 1600, 6400, 1, 0) > 8
    assert tiles.gemm_bf16_splits(72, 1600, 6400, 1, 0) >= 8
    assert 3 <= tiles.gemm_bf16_splits(64, 4800, 1600, 0, 0) <= 8
    assert tiles.gemm_bf16_splits(128, 2304, 768, 0, 0) == 1  # a short K: the second kernel costs more than the walk
    assert tiles.gemm_bf16_splits(512, 2304, 768, 0, 0) == 1
    assert tiles.gemm_bf16_splits(512, 4800, 1600, 0, 0) == 1
    assert tiles.gemm_bf16_splits(2048, 4800, 1600, 0, 0) == 1
    assert 2 <= tiles.gemm_bf16_splits(768, 1600, 6400, 1, 0) <= 4  # a long K pays for a split at more rows
    assert tiles.gemm_bf16_splits(2048, 1600, 6400, 1, 0) == 1
    assert tiles.gemm_bf16_splits(100, 96, 128, 0, 0) == 1  # too few k-blocks to share out
    assert tiles.gemm_bf16_splits(100, 96, 128, 0, 3) == 2


@pytest.mark.parametrize("M", [1, 5, 16, 40, 80])
@pytest.mark.parametrize("dtype,splits", [(torch.bfloat16, None), (torch.bfloat16, 2), (torch.float32, None)])
def test_projection_scatters_keys_and_values(M, dtype, splits):
    """Fused (decode kernels, also with K split and the scatter in the second kernel) and composed
    (general kernels) give the same pages and queries."""
    k = _k()
    H, Hkv, hd, ps, D = 6, 2, 32, 16, 96
    c = PagedCase(dtype, H, Hkv, hd, ps, [30] * M, [1] * M, seed=M)
    qw, kw = H * hd, Hkv * hd
    w = _rand((qw + 2 * kw, D), dtype, 3, 0.2)
    bias = _rand((qw + 2 * kw,), torch.float32, 4, 0.1)
    a = _rand((M, D), dtype, 5)
    ref = plain.linear(a.double().cpu(), w.double().cpu(), bias.double().cpu())
    out = torch.full((M, qw + 2 * kw), float("nan")).to(dtype).to(DEV)
    sc = k.KVScatter(c.kv, c.block_table_dev, c.token_req, c.positions, qw)
    k.linear(out, a, w, bias, scatter=sc, splits=splits)
    torch.cuda.synchronize()
    tol = dict(rtol=2**-7, atol=1e-3) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-5)
    assert torch.allclose(out[:, :qw].double().cpu(), ref[:, :qw], **tol)
    pool = c.pool.cpu()
    for m in range(M):
        page, row = c.block_table[m, 30 // ps], 30 % ps
        assert torch.allclose(pool[page, 0, :, row].reshape(-1).double(), ref[m, qw : qw + kw], **tol)
        assert torch.allclose(pool[page, 1, :, row].reshape(-1).double(), ref[m, qw + kw :], **tol)
        # and nothing else in the page was touched
        assert torch.isnan(pool[page, 0, :, row + 1 :].float()).all()


@pytest.mark.parametrize("variant", [0, 1, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("packed", [False, True])
def test_tile_products_scatter_keys_and_values_themselves(variant, packed):
    """The many-row product writes keys and values into their pages from its own epilogue (every tile
    shape; head size 64 and 80, requests at different positions, rows that are no multiple of a tile,
    a tile that straddles the edge between queries and keys): the same pages as the product followed
    by kv_write, and the key and value columns of the output are left alone."""
    k = _k()
    for H, Hkv, hd, M_per in ((5, 5, 64, [70, 1, 130, 33]), (4, 2, 80, [90, 45])):
        ps, D = 16, 136
        c = PagedCase(torch.bfloat16, H, Hkv, hd, ps, [7 + 20 * i for i in range(len(M_per))], M_per, seed=variant)
        M = sum(M_per)
        qw, kw = H * hd, Hkv * hd
        w = _rand((qw + 2 * kw, D), torch.bfloat16, 3, 0.2)
        bias = _rand((qw + 2 * kw,), torch.float32, 4, 0.1)
        a = _rand((M, D), torch.bfloat16, 5)
        # the product alone, then kv_write (into pages that hold nothing else)
        c.pool.fill_(float("nan"))
        plain_out = torch.empty(M, qw + 2 * kw, dtype=torch.bfloat16, device=DEV)
        k.linear(plain_out, a, w, bias, variant=variant)
        k.kv_write(plain_out[:, qw : qw + kw], plain_out[:, qw + kw :], c.kv, c.block_table_dev, c.token_req, c.positions)
        want_pool = c.pool.clone()
        c.pool.fill_(float("nan"))
        out = torch.full((M, qw + 2 * kw), float("nan"), dtype=torch.bfloat16, device=DEV)
        sc = k.KVScatter(c.kv, c.block_table_dev, c.token_req, c.positions, qw)
        k.linear(out, a, k.PackedWeight(w, keep_rows=False) if packed else w, bias, scatter=sc, variant=variant)
        assert torch.equal(out[:, :qw], plain_out[:, :qw])
        assert torch.isnan(out[:, qw:].float()).all()
        written = ~torch.isnan(want_pool.float())
        assert written.any() and torch.equal(c.pool[written], want_pool[written])
        assert torch.isnan(c.pool[~written].float()).all()
