"""Each kernel of the mixers with a state per row, of attention over a cached latent and of
blocks with norms on both sides, alone against its plain PyTorch counterpart: steps of
several sequences of unequal length (one token, two, many) from a non-zero state, sizes that
are no multiple of the kernels' steps, float32 tightly and bfloat16 against the float32
result of the same bfloat16 inputs."""

from types import SimpleNamespace

import pytest
import torch

from torch_kernels import TorchKernels

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: dict(atol=3e-5, rtol=3e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def kernel_sets():
    from socrates_amd.kernels import HipKernels
    return {dt: (HipKernels(dt, DEV), TorchKernels(dt, DEV)) for dt in DTYPES}


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, dtype, **over):
    torch.testing.assert_close(got.float(), want.float(), **dict(TOL[dtype], **over))


def step_of(lengths, rows):
    """A step's sequences: their starts among the tokens and their state rows."""
    starts = [0]
    for n in lengths:
        starts.append(starts[-1] + n)
    return SimpleNamespace(n_seqs=len(lengths), max_q_len=max(lengths), n_tokens=starts[-1],
                           seq_qstart=torch.tensor(starts, dtype=torch.int32, device=DEV),
                           seq_rows=torch.tensor(rows, dtype=torch.int32, device=DEV))


STEPS = [([1], [0]), ([2, 1, 37], [3, 0, 5]), ([70, 1, 1, 9], [1, 6, 2, 4])]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,d,gated,follows", [(1, 64, True, True), (9, 72, True, False), (5, 2560, False, True), (3, 1001, True, True), (2, 4100, True, False),
                                                (2, 8192, True, True), (2, 9001, True, True)])
def test_gated_norm_add(kernel_sets, dtype, N, d, gated, follows):
    hip, ref = kernel_sets[dtype]
    res, y = rnd((N, d), torch.float32, 1), rnd((N, d), dtype, 2, 0.3)
    logits, bias = (rnd((N, d), dtype, 3), rnd((d,), torch.float32, 4)) if gated else (None, None)
    gain, nxt = rnd((d,), torch.float32, 5), (rnd((d,), torch.float32, 6) if follows else None)
    r1, r2 = res.clone(), res.clone()
    a = hip.gated_norm_add(r1, y, logits, bias, gain, 1e-5, 0.7, nxt, 1e-6)
    b = ref.gated_norm_add(r2, y, logits, bias, gain, 1e-5, 0.7, nxt, 1e-6)
    torch.testing.assert_close(r1, r2, atol=2e-5, rtol=2e-5)
    assert (a is None) == (not follows)
    if follows:
        close(a, b, dtype)
    if gated:
        # the logits as columns of a wider product, at an offset that is a multiple of 8 and at one that is not
        for off in (16, 3):
            wide = rnd((N, off + d + 5), dtype, 7)
            wide[:, off:off + d] = logits
            r3 = res.clone()
            a3 = hip.gated_norm_add(r3, y, wide[:, off:off + d], bias, gain, 1e-5, 0.7, nxt, 1e-6)
            torch.testing.assert_close(r3, r1, atol=1e-6, rtol=1e-6)
            if follows:
                close(a3, a, dtype, atol=1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_glu_clamped(kernel_sets, dtype):
    hip, ref = kernel_sets[dtype]
    for ff in (93, 96, 1000):
        x = rnd((7, 2 * ff), dtype, 1, 2.0)
        close(hip.glu_clamped(x, 1.5, 1.702), ref.glu_clamped(x, 1.5, 1.702), dtype)
        for extra in (8, 13):           # gate and up as the first columns of a wider product
            wide = torch.cat([x, rnd((7, extra), dtype, 2)], dim=1).contiguous()
            close(hip.glu_clamped(wide, 1.5, 1.702, ff), ref.glu_clamped(x, 1.5, 1.702), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lengths,rows", STEPS)
def test_token_shift(kernel_sets, dtype, lengths, rows):
    hip, ref = kernel_sets[dtype]
    d, ctx = 72, step_of(lengths, rows)
    h, mu = rnd((ctx.n_tokens, d), dtype, 1), rnd((5, d), torch.float32, 2)
    s1 = rnd((8, d + 11), torch.float32, 3).to(dtype).float()
    s2 = s1.clone()
    close(hip.token_shift(h, mu, s1, 11, ctx), ref.token_shift(h, mu, s2, 11, ctx), dtype)
    torch.testing.assert_close(s1, s2, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_wkv_decay(kernel_sets, dtype):
    hip, ref = kernel_sets[dtype]
    t, w2, w0 = rnd((6, 24), torch.float32, 1), rnd((24, 200), dtype, 2, 0.3), rnd((200,), torch.float32, 3)
    torch.testing.assert_close(hip.wkv_decay(t, w2, w0), ref.wkv_decay(t, w2, w0), atol=1e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lengths,rows", STEPS)
@pytest.mark.parametrize("H,D", [(3, 16), (2, 40), (2, 64), (1, 144)])
def test_wkv(kernel_sets, dtype, lengths, rows, H, D):
    hip, ref = kernel_sets[dtype]
    ctx, C = step_of(lengths, rows), H * D
    N = ctx.n_tokens
    r, k, v, g = (rnd((N, C), dtype, i, 0.5) for i in range(4))
    decay = torch.rand((N, C), generator=torch.Generator().manual_seed(9)).to(DEV) * 0.5 + 0.5
    bonus, gain = rnd((H, D), torch.float32, 5), rnd((C,), torch.float32, 6)
    s1 = rnd((8, 7 + H * D * D), torch.float32, 7)
    s2 = s1.clone()
    close(hip.wkv(r, k, v, decay, g, bonus, gain, 1e-5, H, s1, 7, ctx), ref.wkv(r, k, v, decay, g, bonus, gain, 1e-5, H, s2, 7, ctx),
          dtype, atol=3e-4 if dtype == torch.float32 else 3e-2)
    torch.testing.assert_close(s1, s2, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lengths,rows", STEPS)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_causal_conv_silu(kernel_sets, dtype, lengths, rows, taps):
    hip, ref = kernel_sets[dtype]
    ctx, C, col = step_of(lengths, rows), 300, 17
    x = rnd((ctx.n_tokens, C + 40), dtype, 1)
    w, b = rnd((C, taps), torch.float32, 2), rnd((C,), torch.float32, 3)
    s1 = rnd((8, 5 + (taps - 1) * C), torch.float32, 4).to(dtype).float()
    s2 = s1.clone()
    close(hip.causal_conv_silu(x, col, C, w, b, s1, 5, ctx), ref.causal_conv_silu(x, col, C, w, b, s2, 5, ctx), dtype)
    torch.testing.assert_close(s1, s2, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lengths,rows", STEPS)
@pytest.mark.parametrize("H,P,Ns,G", [(4, 16, 16, 2), (6, 24, 48, 3), (2, 64, 128, 1), (3, 80, 20, 1)])
def test_ssd(kernel_sets, dtype, lengths, rows, H, P, Ns, G):
    hip, ref = kernel_sets[dtype]
    ctx = step_of(lengths, rows)
    N = ctx.n_tokens
    xbc, dt = rnd((N, H * P + 2 * G * Ns), dtype, 1, 0.5), rnd((N, H), torch.float32, 2)
    dt_bias, a_log, skip = rnd((H,), torch.float32, 3), rnd((H,), torch.float32, 4, 0.5), rnd((H,), torch.float32, 5)
    s1 = rnd((8, 3 + H * Ns * P), torch.float32, 6)
    s2 = s1.clone()
    a = hip.ssd(xbc, dt, dt_bias, a_log, skip, H, P, Ns, G, s1, 3, ctx)
    b = ref.ssd(xbc, dt, dt_bias, a_log, skip, H, P, Ns, G, s2, 3, ctx)
    assert a.dtype == torch.float32
    torch.testing.assert_close(a, b, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(s1, s2, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", [16, 24, 48, 64, 96, 128, 192, 256])
@pytest.mark.parametrize("seqs,H,longest", [(2, 24, 9), (12, 24, 9), (2, 24, 70), (2, 5, 70)])
def test_recurrences_at_every_state_size(kernel_sets, dtype, size, seqs, H, longest):
    """Every size the kernels are built for, in both layouts of a head's columns over workgroups: blocks of 16
    (few heads and sequences, or a prompt portion in the step) and of 64 (many single tokens); sequences of one
    token to ``longest``, from a non-zero state."""
    hip, ref = kernel_sets[dtype]
    lengths = [1 + (3 * i) % 9 for i in range(seqs - 1)] + [longest]
    ctx = step_of(lengths, list(range(seqs)))
    N = ctx.n_tokens
    # wkv: keys and columns of `size`
    C = H * size
    r, k, v, g = (rnd((N, C), dtype, i, 0.5) for i in range(4))
    decay = torch.rand((N, C), generator=torch.Generator().manual_seed(9)).to(DEV) * 0.5 + 0.5
    bonus, gain = rnd((H, size), torch.float32, 5), rnd((C,), torch.float32, 6)
    s1 = rnd((seqs, H * size * size), torch.float32, 7)
    s2 = s1.clone()
    close(hip.wkv(r, k, v, decay, g, bonus, gain, 1e-5, H, s1, 0, ctx), ref.wkv(r, k, v, decay, g, bonus, gain, 1e-5, H, s2, 0, ctx),
          dtype, atol=5e-4 if dtype == torch.float32 else 3e-2)
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)
    # ssd: a state of `size` keys, 40 columns, heads in 3 groups
    P, G = 40, (3 if H % 3 == 0 else 1)
    xbc, dt = rnd((N, H * P + 2 * G * size), dtype, 11, 0.5), rnd((N, H), torch.float32, 12)
    dt_bias, a_log, skip = rnd((H,), torch.float32, 13), rnd((H,), torch.float32, 14, 0.5), rnd((H,), torch.float32, 15)
    s1 = rnd((seqs, H * size * P), torch.float32, 16)
    s2 = s1.clone()
    a = hip.ssd(xbc, dt, dt_bias, a_log, skip, H, P, size, G, s1, 0, ctx)
    b = ref.ssd(xbc, dt, dt_bias, a_log, skip, H, P, size, G, s2, 0, ctx)
    torch.testing.assert_close(a, b, atol=5e-4, rtol=5e-4)
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner,groups", [(96, 1), (96, 3), (1024, 2)])
def test_gated_group_norm(kernel_sets, dtype, inner, groups):
    hip, ref = kernel_sets[dtype]
    y, z, gain = rnd((5, inner), torch.float32, 1), rnd((5, inner + 30), dtype, 2), rnd((inner,), torch.float32, 3)
    close(hip.gated_group_norm(y, z, gain, groups, 1e-5), ref.gated_group_norm(y, z, gain, groups, 1e-5), dtype)


def _latent_slot(dtype, width, block, pages, rows):
    pool = torch.zeros((pages + 1, 1, block, width), dtype=dtype, device=DEV)
    table = torch.randperm(pages)[: rows * (pages // rows)].view(rows, -1).to(torch.int32).to(DEV) + 1
    return SimpleNamespace(k=pool, v=pool, block_table=table, block_size=block, window=None)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("R,Dr,dims,width,block", [(64, 16, 16, 80, 16), (24, 12, 8, 48, 4), (100, 30, 30, 144, 8)])
def test_latent_write_and_query(kernel_sets, dtype, R, Dr, dims, width, block):
    hip, ref = kernel_sets[dtype]
    N, H, D = 11, 3, 20
    s1, s2 = _latent_slot(dtype, width, block, 24, 3), None
    s2 = SimpleNamespace(k=s1.k.clone(), v=None, block_table=s1.block_table, block_size=block, window=None)
    positions = torch.tensor([0, 1, 2, 3, 30, 31, 5, 6, 7, 8, 9], dtype=torch.int32, device=DEV)
    rows = torch.tensor([0, 0, 0, 0, 1, 1, 2, 2, 2, 2, 2], dtype=torch.int32, device=DEV)
    inv_freq = (1e4 ** (-torch.arange(dims // 2, dtype=torch.float64) * 2 / dims)).float().to(DEV)
    kvd, gain = rnd((N, R + Dr), dtype, 1), rnd((R,), torch.float32, 2)
    hip.latent_write(kvd, R, Dr, gain, 1e-5, inv_freq, positions, rows, s1)
    ref.latent_write(kvd, R, Dr, gain, 1e-5, inv_freq, positions, rows, s2)
    close(s1.k, s2.k, dtype)
    # the same rows as columns of a wider product
    wide = rnd((N, 7 + R + Dr + 3), dtype, 9)
    wide[:, 7:7 + R + Dr] = kvd
    s3 = SimpleNamespace(k=torch.zeros_like(s1.k), v=None, block_table=s1.block_table, block_size=block, window=None)
    hip.latent_write(wide[:, 7:7 + R + Dr], R, Dr, gain, 1e-5, inv_freq, positions, rows, s3)
    torch.testing.assert_close(s3.k, s1.k, atol=0, rtol=0)
    close(hip.rmsnorm_cols(wide[:, 7:7 + R], gain, 1e-5), ref.rmsnorm_cols(kvd[:, :R], gain, 1e-5), dtype)
    q, w = rnd((N, H * (D + Dr)), dtype, 3), rnd((H, R, D), dtype, 4, 0.3)
    close(hip.latent_query(q, H, D, Dr, w, width, inv_freq, positions), ref.latent_query(q, H, D, Dr, w, width, inv_freq, positions),
          dtype, atol=5e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,H,ldx,K,n_out", [(1, 1, 16, 16, 16), (8, 20, 160, 128, 96), (16, 3, 80, 70, 33), (17, 3, 80, 70, 33), (19, 5, 80, 64, 70),
                                             (70, 2, 144, 100, 129)])
def test_head_project(kernel_sets, dtype, N, H, ldx, K, n_out):
    hip, ref = kernel_sets[dtype]
    x, w = rnd((N, H, ldx), dtype, 1), rnd((H, n_out, K), dtype, 2, 0.2)
    close(hip.head_project(x, w), ref.head_project(x, w), dtype, atol=5e-5 if dtype == torch.float32 else 3e-2)
