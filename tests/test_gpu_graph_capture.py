"""The operators under HIP graph capture.  The library allocates nothing, clears nothing with memset nodes and never
synchronises, so a serving loop can record a decode step (rotary, KV write, both decode stages) or a prefill step once and
replay it.  Each graph is replayed several times on new inputs, with eager work and synchronisations between the
replays, and every replay is compared with the eager result of the same operators."""
import pytest
import torch

from tests.helpers import decode_case, meta, rand_t

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("kernel", ["the library's choice", "matrix pipe"])
def test_decode_step_replays_match_eager(lsa, tuning, kernel):
    if kernel == "matrix pipe":  # (a launch this small takes the lane kernel by itself)
        tuning(decode_stage1="mfma")
    B, Hq, Hkv, D, BS = 4, 8, 2, 128, 64
    pool, max_len = 4000, 900
    _, kv, _, _, _ = decode_case(300, B, Hq, Hkv, D, [1] * B, pool)
    kv0 = kv.to(DEV)
    nblk = (max_len + BS - 1) // BS

    def buffers():
        return dict(q=torch.zeros(B, Hq, D, dtype=torch.float16, device=DEV),
                    kv_new=torch.zeros(B, 2 * Hkv, D, dtype=torch.float16, device=DEV),
                    cos=torch.zeros(B, D // 2, dtype=torch.float16, device=DEV),
                    sin=torch.zeros(B, D // 2, dtype=torch.float16, device=DEV),
                    new_slots=torch.zeros(B, dtype=torch.int32, device=DEV),
                    table=torch.zeros(B + 2, max_len + 5, dtype=torch.int32, device=DEV),
                    b_req=torch.zeros(B, dtype=torch.int32, device=DEV),
                    b_len=torch.ones(B, dtype=torch.int32, device=DEV),
                    pool=kv0.clone(),
                    mid_o=torch.empty(nblk, B, Hq, D, dtype=torch.float32, device=DEV),
                    mid_l=torch.empty(nblk, B, Hq, dtype=torch.float32, device=DEV),
                    o=torch.empty(B, Hq, D, dtype=torch.float32, device=DEV),
                    lse=torch.empty(B, Hq, dtype=torch.float32, device=DEV))

    def step(s):
        lsa.longserve_cuda_kernels.rotary_emb(s["q"], s["kv_new"][:, :Hkv], s["cos"], s["sin"])
        lsa.kv_scatter(s["kv_new"], s["new_slots"], s["pool"])
        lsa.longserve_token_decode_attention_flash_decoding(
            s["q"], s["table"], s["b_req"], s["b_len"], s["mid_o"], s["mid_l"], B, max_len, Hq, D,
            s["pool"][:, :Hkv], s["pool"][:, Hkv:], BS, out=s["o"], o_logexpsum=s["lse"])

    def fill(s, seed, lens):
        q, _, table, b_req, b_len = decode_case(seed, B, Hq, Hkv, D, lens, pool, pad_seq=max_len + 5 - max(lens))
        g = torch.Generator().manual_seed(seed)
        s["q"].copy_(q)
        s["kv_new"].copy_(rand_t((B, 2 * Hkv, D), seed + 7))
        ang = torch.rand(B, D // 2, generator=g) * 6.0
        s["cos"].copy_(torch.cos(ang).half()); s["sin"].copy_(torch.sin(ang).half())
        s["table"].copy_(table); s["b_req"].copy_(b_req); s["b_len"].copy_(b_len)
        # the new token of request b sits in the last registered slot of its row
        last = torch.stack([table[int(b_req[b]), lens[b] - 1] for b in range(B)])
        s["new_slots"].copy_(last)

    cases = [(310, [900, 64, 65, 1]), (320, [5, 700, 128, 333]), (330, [1, 1, 2, 63])]
    st = buffers()
    fill(st, *cases[0])
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(st)
    for seed, lens in cases + cases[:1]:
        print("decode replay", seed, lens, flush=True)
        fill(st, seed, lens)
        graph.replay()
        torch.cuda.synchronize()
        eager = buffers()
        fill(eager, seed, lens)
        step(eager)
        torch.cuda.synchronize()
        assert torch.equal(st["q"], eager["q"])
        assert torch.equal(st["o"], eager["o"]) and torch.equal(st["lse"], eager["lse"])
        rows = st["new_slots"].long()
        assert torch.equal(st["pool"][rows], eager["pool"][rows])
        st["pool"].copy_(kv0)   # each case starts from the same pool contents, as the eager run does


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_step_replays_match_eager(lsa, dtype):
    Hq, Hkv, D = 4, 2, 128
    lens = [700, 300]
    T = sum(lens)
    sd, bd, fd = [t.to(DEV) for t in meta(lens)]
    # (bfloat16: the fp16 copy of V is a torch allocation of the Python operator; it is made once, at capture, from the
    # caching allocator's graph pool, and the replays write the same memory)

    def buffers():
        return dict(q=torch.zeros(T, Hq, D, dtype=dtype, device=DEV), k=torch.zeros(T, Hkv, D, dtype=dtype, device=DEV),
                    v=torch.zeros(T, Hkv, D, dtype=dtype, device=DEV), o=torch.zeros(T, Hq, D, dtype=dtype, device=DEV),
                    m=torch.zeros(T, Hq, device=DEV), l=torch.zeros(T, Hq, device=DEV),
                    po=torch.zeros(T, Hq, D, device=DEV), plse=torch.zeros(T, Hq, device=DEV))

    def step(s):
        s["m"].fill_(float("-inf")); s["l"].zero_()
        lsa.context_attention_fwd(s["q"], s["k"], s["v"], s["o"], sd, bd, fd, sd, bd, fd, 1, max(lens), s["m"], s["l"])
        lsa.prefill_attention_step(s["q"], s["k"], s["v"], sd, bd, fd, sd, bd, fd, 1, max(lens), out=s["po"], lse=s["plse"])

    def fill(s, seed):
        s["q"].copy_(rand_t((T, Hq, D), seed, dtype)); s["k"].copy_(rand_t((T, Hkv, D), seed + 1, dtype))
        s["v"].copy_(rand_t((T, Hkv, D), seed + 2, dtype))

    st = buffers()
    fill(st, 400)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(st)
    for seed in (400, 410, 420, 400):
        print("prefill replay", dtype, seed, flush=True)
        fill(st, seed)
        graph.replay()
        torch.cuda.synchronize()
        eager = buffers()
        fill(eager, seed)
        step(eager)
        torch.cuda.synchronize()
        for name in ("o", "m", "l", "po", "plse"):
            assert torch.equal(st[name], eager[name]), name
