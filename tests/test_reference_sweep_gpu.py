"""The reference harness's own sweep (test_pa_mtp.py:48-55: block sizes 16/64/1024, head configurations
(5,1) (8,1) (10,1) (16,1) (64,4), query lengths 1..4, context lengths 512/4096/4097, both V layouts), at its
smallest batch size (4), with inputs made the way the harness makes them (test_pa_mtp.py:690-722,763-783):
uniform(-1,1) bf16 query and cache, block tables drawn WITH replacement from the pool (pages alias within and
across sequences), the cache quantised per (block, head, token) on the GPU, the query per row.

Each configuration is run three ways, as the harness does: the 16-bit cache, the FP8 cache under the bf16 query,
and the FP8 cache under the FP8 query with its per-row scales (the Gluon entry point's contract).  The bar is the
CPU oracle on the same bytes at atol = rtol = 2e-2 (the harness itself checks at 5e-2).  The partition size is
the library's own choice, so the sweep covers the default path end to end.
"""
import pytest
import torch

from oracle import pa_oracle as O

pytestmark = pytest.mark.gpu

ATOL = RTOL = 2e-2
HEAD_CONFIGURATIONS = [(5, 1), (8, 1), (10, 1), (16, 1), (64, 4)]
BATCH = 4


@pytest.mark.parametrize("trans_v", [False, True], ids=["plainV", "transV"])
@pytest.mark.parametrize("q_len", [1, 2, 3, 4])
@pytest.mark.parametrize("heads", HEAD_CONFIGURATIONS, ids=lambda h: f"h{h[0]}x{h[1]}")
@pytest.mark.parametrize("block_size", [16, 64, 1024])
def test_reference_sweep_configuration(cuda, block_size, heads, q_len, trans_v):
    import triton_op_amd as T
    from triton_op_amd import kv_layout as L

    hq, hkv = heads
    d = 128
    gen = torch.Generator().manual_seed(1000 * block_size + 10 * hq + q_len)
    blocks_per_seq = (4097 + block_size - 1) // block_size
    pool = BATCH * blocks_per_seq * 5 // 4
    kc16, vc16 = L.create_kv_cache(pool, block_size, hkv, d, torch.bfloat16, generator=gen)
    block_tables = torch.randint(0, pool, (BATCH, blocks_per_seq), generator=gen, dtype=torch.int32)
    q_tok = torch.empty(BATCH * q_len, hq, d).uniform_(-1.0, 1.0, generator=gen).to(torch.bfloat16)
    query = L.mtp_pack(q_tok, BATCH, q_len, hkv).contiguous()
    scale = 1.0 / d ** 0.5

    kq, _, vq, _, ks, vs = T.quantize_kv_cache_symmetric(kc16.to(cuda), vc16.to(cuda), torch.float8_e4m3fn)
    q8, q8s = L.pertoken_quant(query.float())
    caches = {
        "bf16": (kc16, vc16, None, None),
        "fp8": (kq.cpu(), vq.cpu(), ks.cpu(), vs.cpu()),
    }
    dev = {}
    for k, (kc, vc, s1, s2) in caches.items():
        v_op = L.shuffle_value_cache_layout(vc) if trans_v else vc
        dev[k] = (kc.to(cuda), v_op.to(cuda), None if s1 is None else s1.to(cuda), None if s2 is None else s2.to(cuda))
    bt_dev = block_tables.to(cuda)

    for ctx in (512, 4096, 4097):
        lens = torch.full((BATCH,), ctx, dtype=torch.int32)
        lens_dev = lens.to(cuda)
        for leg in ("bf16", "fp8", "fp8_q8"):
            print(f"block_size={block_size} heads={heads} q_len={q_len} trans_v={trans_v} ctx={ctx} leg={leg}", flush=True)
            kc, vc, s1, s2 = caches["bf16" if leg == "bf16" else "fp8"]
            kcd, vcd, s1d, s2d = dev["bf16" if leg == "bf16" else "fp8"]
            q_in, qs_in = (q8, q8s) if leg == "fp8_q8" else (query, None)
            out = torch.full((BATCH, hkv * q_len * (hq // hkv), d), float("nan"), dtype=torch.bfloat16, device=cuda)
            T.paged_attention_decode(out, q_in.to(cuda), kcd, vcd, lens_dev, bt_dev, scale, q_len, ctx, torch.bfloat16,
                                     None if qs_in is None else qs_in.to(cuda), s1d, s2d)
            torch.cuda.synchronize()
            ref = O.paged_attention_decode_oracle(q_in, kc, vc, lens, block_tables, scale, q_len, s1, s2,
                                                  query_scale=qs_in)
            assert not torch.isnan(out.float()).any()
            torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
