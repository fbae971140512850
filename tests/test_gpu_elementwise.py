"""GPU parity of rms_norm / silu_and_mul_inplace / rotary_emb / ffn_block against the numpy oracle (through the C ABI).

Tolerances: rotary_emb is bit-exact (the kernel performs the reference's half operations one by one).  rms_norm and
silu_and_mul round an fp32 value to half: a different summation order / exp implementation may move a value across a
rounding boundary, so results may differ from the oracle by one fp16 step (two after silu's extra half multiply); asserted: never more,
and on few elements."""
import numpy as np
import pytest
import torch

from oracle import elementwise_oracle as ew

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ulp(a, b):
    def key(v):
        i = v.view(np.int16).astype(np.int32)
        return np.where(i < 0, -32768 - i, i)
    return np.abs(key(a) - key(b))


@pytest.mark.parametrize("T,H", [(1, 8), (5, 4096), (131, 5120), (3, 8192), (2, 8200), (4, 16384)])
def test_rms_norm(lsa, T, H):
    rng = np.random.default_rng(T * 31 + H)
    x = (rng.standard_normal((T, H)) * 1.5).astype(np.float16)
    w = (1 + 0.2 * rng.standard_normal(H)).astype(np.float16)
    out = lsa.longserve_cuda_kernels.rms_norm(torch.from_numpy(x).to(DEV), torch.from_numpy(w).to(DEV), 1e-5)
    torch.cuda.synchronize()
    got, want = out.cpu().numpy(), ew.rms_norm(x, w, 1e-5)
    d = _ulp(got, want)
    assert d.max() <= 1 and (d > 0).mean() < 2e-2, (d.max(), (d > 0).mean())
    # the name the post layer calls for the final norm takes any leading shape (models/llama/triton_kernel/rmsnorm.py:41)
    x3 = torch.from_numpy(x).to(DEV).view(1, T, H)
    out3 = lsa.rmsnorm_forward(x3, torch.from_numpy(w).to(DEV), 1e-5)
    assert out3.shape == x3.shape and torch.equal(out3.view(T, H), out)


@pytest.mark.parametrize("T,I", [(1, 8), (7, 11008), (64, 13824), (3, 1000)])
def test_silu_and_mul_inplace(lsa, T, I):
    rng = np.random.default_rng(T + I)
    io = (rng.standard_normal((T, 2 * I)) * 3).astype(np.float16)
    d_io = torch.from_numpy(io).to(DEV)
    lsa.longserve_cuda_kernels.silu_and_mul_inplace(d_io)
    torch.cuda.synchronize()
    want = io.copy()
    ew.silu_and_mul_inplace(want)
    got = d_io.cpu().numpy()
    assert np.array_equal(got[:, I:], io[:, I:])  # the up half is untouched
    # silu is rounded to half and then multiplied in half: when the fp32 silu (v_exp_f32, ~1e-7 relative) lands on the
    # other side of a half rounding boundary than the float64 oracle (probability ~1e-3), the product moves by one step,
    # or two across a binade; never more
    d = _ulp(got[:, :I], want[:, :I])
    assert d.max() <= 2 and (d > 0).mean() < 2e-3, (d.max(), (d > 0).mean())


@pytest.mark.parametrize("T,Hq,Hkv,D", [(1, 1, 1, 16), (33, 32, 8, 128), (200, 10, 5, 64), (5, 4, 4, 256)])
def test_rotary_emb_bit_exact_on_strided_views(lsa, T, Hq, Hkv, D):
    rng = np.random.default_rng(T * 7 + D)
    qkv = rng.standard_normal((T, Hq + 2 * Hkv, D)).astype(np.float16)   # q and k are strided views of one buffer (as in the model)
    ang = rng.uniform(0, 6.28, (T, D // 2))
    cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
    d = torch.from_numpy(qkv).to(DEV)
    lsa.longserve_cuda_kernels.rotary_emb(d[:, :Hq], d[:, Hq:Hq + Hkv], torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV))
    torch.cuda.synchronize()
    want = qkv.copy()
    ew.rotary_emb(want[:, :Hq], cos, sin)
    ew.rotary_emb(want[:, Hq:Hq + Hkv], cos, sin)
    assert np.array_equal(d.cpu().numpy().view(np.int16), want.view(np.int16))   # v heads untouched, q/k bit-exact


@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("Hq,Hkv,D", [(32, 8, 128), (4, 4, 64), (6, 1, 32)])
def test_fused_rotary_kv_write_register_matches_the_separate_operators(lsa, decode, Hq, Hkv, D):
    """lsattn_rotary_kv_write against the oracles of the three steps it replaces: rotary of q and k (bit-exact), the
    rotated K rows and the V rows in their pool slots (bit-exact row scatter), and the request table (prefill: every
    token of every request; decode: the last token of every request)."""
    from oracle import attn_oracle as orc
    rng = np.random.default_rng(Hq * 13 + D + decode)
    lens = [5, 1, 40, 17] if not decode else [9, 300, 1, 64, 2]
    B = len(lens)
    T = B if decode else sum(lens)
    qkv = rng.standard_normal((T, Hq + 2 * Hkv, D)).astype(np.float16)   # q and kv are views of one buffer, as in the model
    ang = rng.uniform(0, 6.28, (T, D // 2))
    cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
    slots = 3 * T + 7
    g = torch.Generator().manual_seed(5)
    mem_index = torch.randperm(slots, generator=g)[:T].to(torch.int32)
    pool0 = torch.from_numpy(rng.standard_normal((slots, 2 * Hkv, D)).astype(np.float16))
    max_seq = max(lens) + 3
    table0 = torch.full((B + 2, max_seq), orc.INT32_PAD, dtype=torch.int32)
    b_req = torch.randperm(B + 2, generator=g)[:B].to(torch.int32)
    b_len = torch.tensor(lens, dtype=torch.int32)
    b_start = (torch.cumsum(b_len, 0) - b_len).to(torch.int32)
    d = torch.from_numpy(qkv).to(DEV)
    pool, table = pool0.clone().to(DEV), table0.clone().to(DEV)
    lsa.rotary_emb_write_kv(d[:, :Hq], d[:, Hq:], torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV), mem_index.to(DEV), pool,
                            table, b_req.to(DEV), b_len.to(DEV), None if decode else b_start.to(DEV), None if decode else max(lens),
                            decode=decode)
    torch.cuda.synchronize()
    want = qkv.copy()
    ew.rotary_emb(want[:, :Hq], cos, sin)
    ew.rotary_emb(want[:, Hq:Hq + Hkv], cos, sin)
    assert np.array_equal(d.cpu().numpy().view(np.int16), want.view(np.int16))          # q, k rotated in place, v untouched
    pool_ref, table_ref = pool0.clone(), table0.clone()
    orc.kv_scatter(torch.from_numpy(want[:, Hq:].copy()), mem_index, pool_ref)
    if decode:
        orc.copy_kv_index_to_req(table_ref, b_req, b_len, mem_index)
    else:
        orc.register_tokens(table_ref, b_req, b_start, b_len, mem_index)
    assert torch.equal(pool.cpu().view(torch.int16), pool_ref.view(torch.int16))         # every slot: written rows and the rest
    assert torch.equal(table.cpu(), table_ref)
    # without a pool and without a table it is the rotary step alone
    d2 = torch.from_numpy(qkv).to(DEV)
    lsa.rotary_emb_write_kv(d2[:, :Hq], d2[:, Hq:], torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(d2.cpu().numpy().view(np.int16), want.view(np.int16))


def test_ffn_block_composition(lsa):
    rng = np.random.default_rng(9)
    T, H, I = 17, 512, 1024
    x = (rng.standard_normal((T, H))).astype(np.float16)
    nw = (1 + 0.1 * rng.standard_normal(H)).astype(np.float16)
    gu = (rng.standard_normal((H, 2 * I)) * 0.05).astype(np.float16)
    dn = (rng.standard_normal((I, H)) * 0.05).astype(np.float16)
    t = lambda a: torch.from_numpy(a).to(DEV)
    out = lsa.longserve_cuda_kernels.ffn_block(t(x), t(nw), 1e-5, t(gu), t(dn))
    torch.cuda.synchronize()
    # float64 restatement of ENTRY:91-101 with the fp16 roundings of the intermediate tensors
    normed = ew.rms_norm(x, nw, 1e-5)
    ug = (normed.astype(np.float64) @ gu.astype(np.float64)).astype(np.float16)
    ew.silu_and_mul_inplace(ug)
    want = ug[:, :I].astype(np.float64) @ dn.astype(np.float64)
    err = np.abs(out.cpu().numpy().astype(np.float64) - want).max()
    assert err <= 2e-2 * max(1.0, np.abs(want).max()), err   # library GEMM accumulation order + fp16 outputs


def test_triton_operator_names_run_the_same_kernels(lsa):
    """rotary_emb_fwd / silu_and_mul_fwd (the Triton duplicates in the reference's tree) give what the extension-module
    functions give, with the Triton wrappers' return convention."""
    g = torch.Generator().manual_seed(3)
    T, Hq, Hkv, D, I = 33, 4, 2, 128, 256
    q = (torch.randn(T, Hq, D, generator=g)).half().to(DEV)
    k = (torch.randn(T, Hkv, D, generator=g)).half().to(DEV)
    ang = torch.rand(T, D // 2, generator=g) * 6
    cos, sin = torch.cos(ang).half().to(DEV), torch.sin(ang).half().to(DEV)
    q2, k2 = q.clone(), k.clone()
    lsa.longserve_cuda_kernels.rotary_emb(q, k, cos, sin)
    assert lsa.rotary_emb_fwd(q2, k2, cos, sin) is None
    assert torch.equal(q, q2) and torch.equal(k, k2)
    io = (torch.randn(T, 2 * I, generator=g) * 2).half().to(DEV)
    io2 = io.clone()
    lsa.longserve_cuda_kernels.silu_and_mul_inplace(io)
    out = lsa.silu_and_mul_fwd(io2)
    assert out.shape == (T, I) and out.data_ptr() == io2.data_ptr() and torch.equal(io, io2)


def test_argument_checks(lsa):
    k = lsa.longserve_cuda_kernels
    with pytest.raises(ValueError):
        k.rms_norm(torch.zeros(2, 8, dtype=torch.float32, device=DEV), torch.zeros(8, dtype=torch.float16, device=DEV), 1e-5)
    with pytest.raises(ValueError):
        k.silu_and_mul_inplace(torch.zeros(2, 8, dtype=torch.float16))  # CPU tensor
    with pytest.raises(RuntimeError):
        k.rms_norm(torch.zeros(2, 12, dtype=torch.float16, device=DEV), torch.zeros(12, dtype=torch.float16, device=DEV), 1e-5)  # 12 % 8 != 0
