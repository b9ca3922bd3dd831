"""The KV-cache write / quantise kernels against the torch formulas in kv_layout (same scale = amax/448,
same float32 division, round to nearest even): the bytes and the scales must match exactly, and a cache
written by the kernels must decode to the same attention output as one built on the host."""
import pytest
import torch

from triton_op_amd import kv_layout as L

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bs,nblk,h", [(16, 37, 2), (64, 5, 3), (1024, 2, 1)])
def test_quantize_whole_cache_matches_torch_bit_for_bit(cuda, bs, nblk, h):
    import triton_op_amd as T

    g = torch.Generator().manual_seed(bs)
    kc, vc = L.create_kv_cache(nblk, bs, h, 128, torch.bfloat16, generator=g, distribution="normal")
    kc[1, 0, :, 3] = 0  # an all-zero key row: scale 1, bytes 0
    kq_ref, ks_ref, vq_ref, vs_ref = L.quantize_kv_cache_per_token(kc, vc)
    kq, ksf, vq, vsf, ks, vs = T.quantize_kv_cache_symmetric(kc.to(cuda), vc.to(cuda), torch.float8_e4m3fn)
    torch.cuda.synchronize()
    assert torch.equal(ks.cpu(), ks_ref) and torch.equal(vs.cpu(), vs_ref)
    assert torch.equal(kq.cpu().view(torch.uint8), kq_ref.view(torch.uint8))
    assert torch.equal(vq.cpu().view(torch.uint8), vq_ref.view(torch.uint8))
    assert float(ks[1, 0, 3, 0]) == 1.0
    assert ksf.shape == (h, nblk * bs) and torch.equal(ksf.cpu(), ks_ref.permute(1, 0, 2, 3).reshape(h, nblk * bs))
    assert torch.equal(vsf.cpu(), vs_ref.permute(1, 0, 2, 3).reshape(h, nblk * bs))


@pytest.mark.parametrize("d", [128, 64, 256], ids=["head128", "head64", "head256"])
@pytest.mark.parametrize("trans_v", [False, True], ids=["plainV", "transV"])
@pytest.mark.parametrize("mode", ["token", "tensor", "bf16"])
def test_cache_write_then_decode(cuda, mode, trans_v, d):
    """Tokens appended through kv_cache_write (in two calls, scattered slots, one padding token) give the same
    cache bytes as the host-side quantiser, and the decode op reads them back correctly; head sizes 64 and 256 take
    the generic kernels of both."""
    import triton_op_amd as T
    from oracle import pa_oracle as O

    bs, nblk, h = 16, 24, 2
    ctx = torch.tensor([70, 133], dtype=torch.int32)
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    bt = perm[:18].view(2, 9).contiguous()
    toks = int(ctx.sum())
    key = torch.randn(toks, h, d, generator=g).to(torch.bfloat16)
    value = torch.randn(toks, h, d, generator=g).to(torch.bfloat16)
    slots = torch.cat([bt[b].long().repeat_interleave(bs)[:int(ctx[b])] * bs + torch.arange(int(ctx[b])) % bs for b in range(2)])
    # host reference cache
    k_tok = torch.zeros(nblk, bs, h, d, dtype=torch.bfloat16)
    v_tok = torch.zeros(nblk, bs, h, d, dtype=torch.bfloat16)
    k_tok.view(-1, h, d)[slots] = key
    v_tok.view(-1, h, d)[slots] = value
    kc16, vc16 = L.tokens_to_key_cache(k_tok), L.tokens_to_value_cache(v_tok)
    dev = cuda
    if mode == "bf16":
        kc = torch.zeros_like(kc16, device=dev)
        vc = torch.zeros_like(vc16, device=dev)
        ks = vs = None
        kref, vref, ksr, vsr = kc16, vc16, None, None
    else:
        kc = torch.zeros(nblk, h, d // 16, bs, 16, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        vc = torch.zeros(nblk, h, d, bs, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        if mode == "token":
            kref, ksr, vref, vsr = L.quantize_kv_cache_per_token(kc16, vc16)
            ks = torch.ones(nblk, h, bs, 1, device=dev)
            vs = torch.ones(nblk, h, bs, 1, device=dev)
        else:
            ksr = (key.float().abs().max() / 448.0).to(torch.float32)
            vsr = (value.float().abs().max() / 448.0).to(torch.float32)
            kref = L.tokens_to_key_cache((k_tok.float() / ksr).to(torch.float8_e4m3fn))
            vref = L.tokens_to_value_cache((v_tok.float() / vsr).to(torch.float8_e4m3fn))
            ks, vs = ksr.to(dev), vsr.to(dev)
    if trans_v:  # the kernel writes (and the decode op reads) the transposed V layout
        vc = L.shuffle_value_cache_layout(vc)
    # append in two calls; the second carries a padding token (slot -1)
    cut = 90
    T.kv_cache_write(key[:cut].to(dev), value[:cut].to(dev), kc, vc, slots[:cut].to(dev), ks, vs)
    k2 = torch.cat([key[cut:], key[:1]]).to(dev)
    v2 = torch.cat([value[cut:], value[:1]]).to(dev)
    s2 = torch.cat([slots[cut:], torch.tensor([-1])]).to(dev)
    T.kv_cache_write(k2, v2, kc, vc, s2, ks, vs)
    torch.cuda.synchronize()
    view = torch.uint8 if mode != "bf16" else torch.int16
    assert torch.equal(kc.cpu().view(view), kref.view(view))
    vplain = L.unshuffle_value_cache_layout(vc) if trans_v else vc
    assert torch.equal(vplain.cpu().view(view), vref.view(view))
    if mode == "token":
        live = torch.zeros(nblk * bs, dtype=torch.bool)
        live[slots] = True
        live = live.view(nblk, 1, bs, 1).expand(nblk, h, bs, 1)
        assert torch.equal(ks.cpu()[live], ksr[live]) and torch.equal(vs.cpu()[live], vsr[live])
        assert bool((ks.cpu()[~live] == 1).all())  # untouched
    # decode from the cache the kernels wrote
    q = torch.randn(2, 16, d, generator=g).to(torch.bfloat16)
    out = torch.empty(2, 16, d, dtype=torch.bfloat16, device=dev)
    T.paged_attention_decode(out, q.to(dev), kc, vc, ctx.to(dev), bt.to(dev), d ** -0.5, 1, 133, torch.bfloat16, None, ks, vs)
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(q, kref, vref, ctx, bt, d ** -0.5, 1, ksr, vsr)
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=2e-2, rtol=2e-2)


def _prefill_like_slots(bs, gen):
    """A token stream that mixes what a serving engine sends: whole prompts of odd lengths (runs that start a
    page), continuations of earlier chunks (runs that start in the middle of a page, also in the middle of a
    16-slot segment), a stretch of single scattered tokens (decode rows), and padding tokens (slot -1)."""
    runs = []  # (first slot, length) or (-1, length) for padding
    page = 0

    def new_pages(n):
        nonlocal page
        first = page
        page += n
        return first

    for length in (1, 15, 16, 17, 100, 333, 1024, 31, 640):  # prompts from the start of a page
        p = new_pages((length + bs - 1) // bs)
        runs.append((p * bs, length))
    for start, length in ((5, 40), (bs - 1, 18), (16 % bs, 200), (9, 3)):  # continuations at an offset
        p = new_pages((start + length + bs - 1) // bs)
        runs.append((p * bs + start, length))
    runs.append((-1, 3))
    for _ in range(70):  # scattered single tokens, every one in a page of its own
        p = new_pages(1)
        runs.append((p * bs + int(torch.randint(0, bs, (1,), generator=gen)), 1))
    runs.append((-1, 1))
    for length in (48, 7, 512):
        p = new_pages((length + bs - 1) // bs)
        runs.append((p * bs, length))
    order = torch.randperm(page, generator=gen)  # the pages are handed out in random order
    slots = []
    for first, length in runs:
        if first < 0:
            slots.append(torch.full((length,), -1, dtype=torch.int64))
            continue
        s = first + torch.arange(length)
        slots.append(order[s // bs] * bs + s % bs)
    return torch.cat(slots), page


@pytest.mark.parametrize("trans_v", [False, True], ids=["plainV", "transV"])
@pytest.mark.parametrize("bs", [16, 64, 1024])
@pytest.mark.parametrize("mode", ["token", "tensor", "bf16"])
def test_cache_write_of_many_tokens_matches_the_host_quantiser(cuda, mode, bs, trans_v):
    """Thousands of tokens in one call take the kernel that writes runs of tokens 16 at a time: every run shape
    (aligned, offset, shorter than 16, crossing pages, scattered, padding) must give the bytes and scales of the
    host-side quantiser, and must leave every other slot of the cache untouched."""
    import triton_op_amd as T

    h, d = 3, 128
    g = torch.Generator().manual_seed(100 + bs)
    slots, nblk = _prefill_like_slots(bs, g)
    toks = slots.numel()
    assert toks >= 2048
    live = slots >= 0
    key = torch.randn(toks, h, d, generator=g).to(torch.bfloat16)
    value = torch.randn(toks, h, d, generator=g).to(torch.bfloat16)
    key[7, 1] = 0  # an all-zero row: scale 1, bytes 0
    if mode == "token":  # rows of extreme magnitude: scales outside and inside the range of the short division
        key[11, 0] *= 1e30
        value[12, 2] *= 1e-30
        key[13, 1] *= 1e-20
        key[13, 1, 5] = 1e20
        value[14, 0] *= 1e9
        key[15, 2] *= 1e-9
    fill = 0.5  # what the cache holds before the call
    k_tok = torch.full((nblk, bs, h, d), fill, dtype=torch.bfloat16)
    v_tok = torch.full((nblk, bs, h, d), fill, dtype=torch.bfloat16)
    k_tok.view(-1, h, d)[slots[live]] = key[live]
    v_tok.view(-1, h, d)[slots[live]] = value[live]
    kc16, vc16 = L.tokens_to_key_cache(k_tok), L.tokens_to_value_cache(v_tok)
    written = torch.zeros(nblk * bs, dtype=torch.bool)
    written[slots[live]] = True
    wk = written.view(nblk, 1, 1, bs, 1)
    wv = written.view(nblk, 1, 1, bs)
    if mode == "bf16":
        kref, vref = kc16, vc16
        kc, vc = torch.full_like(kc16, fill).to(cuda), torch.full_like(vc16, fill).to(cuda)
        ks = vs = None
    else:
        if mode == "token":
            kref, ksr, vref, vsr = L.quantize_kv_cache_per_token(kc16, vc16)
            ks = torch.full((nblk, h, bs, 1), 7.0, device=cuda)
            vs = torch.full((nblk, h, bs, 1), 7.0, device=cuda)
        else:
            ksr = (key.float().abs().max() / 448.0).to(torch.float32)
            vsr = (value.float().abs().max() / 448.0).to(torch.float32)
            kref = L.tokens_to_key_cache((k_tok.float() / ksr).to(torch.float8_e4m3fn))
            vref = L.tokens_to_value_cache((v_tok.float() / vsr).to(torch.float8_e4m3fn))
            ks, vs = ksr.to(cuda), vsr.to(cuda)
        kc = torch.full(kref.shape, 0x55, dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
        vc = torch.full(vref.shape, 0x55, dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
    if trans_v:  # the kernel writes the transposed V layout; it is turned back for the comparison
        vc = L.shuffle_value_cache_layout(vc)
    T.kv_cache_write(key.to(cuda), value.to(cuda), kc, vc, slots.to(cuda), ks, vs)
    torch.cuda.synchronize()
    if trans_v:
        vc = L.unshuffle_value_cache_layout(vc)
    view = torch.uint8 if mode != "bf16" else torch.int16
    kgot, vgot = kc.cpu().view(view), vc.cpu().view(view)
    kexp, vexp = kref.view(view).clone(), vref.view(view).clone()
    before = 0x55 if mode != "bf16" else int(torch.tensor(fill, dtype=torch.bfloat16).view(torch.int16))
    kexp[~wk.expand_as(kexp)] = before
    vexp[~wv.expand_as(vexp)] = before
    assert torch.equal(kgot, kexp)
    assert torch.equal(vgot, vexp)
    if mode == "token":
        w = written.view(nblk, 1, bs, 1).expand(nblk, h, bs, 1)
        assert torch.equal(ks.cpu()[w], ksr[w]) and torch.equal(vs.cpu()[w], vsr[w])
        assert bool((ks.cpu()[~w] == 7.0).all()) and bool((vs.cpu()[~w] == 7.0).all())
        assert float(ks[int(slots[7]) // bs, 1, int(slots[7]) % bs, 0]) == 1.0


@pytest.mark.parametrize("scale_bits", [0x3C7FFFFF, 0x3C800001, 0x3D7FFF80, 0x3DABCDEF, 0x2A800000, 0x55123456],
                         ids=["all_ones", "one_ulp_over_pow2", "high_significand", "generic", "tiny", "huge"])
def test_cache_write_with_awkward_per_tensor_scales(cuda, scale_bits):
    """A caller's per-tensor scale can be any float: the short division of the many-token kernel (one reciprocal,
    one quotient correction; full division for a significand of all ones or a scale outside 2^-40 .. 2^40) must
    give the bytes of the torch formula for rows full of powers of two, near-ties and ordinary values."""
    import triton_op_amd as T

    bs, h, d, toks = 16, 2, 128, 2048
    g = torch.Generator().manual_seed(scale_bits & 0xffff)
    scale = torch.tensor([scale_bits], dtype=torch.int32).view(torch.float32)[0]
    key = (torch.randn(toks, h, d, generator=g) * scale * 100).to(torch.bfloat16)
    value = (torch.randn(toks, h, d, generator=g) * scale * 100).to(torch.bfloat16)
    # powers of two and every fp8 midpoint times the scale (rounded to bf16): where a quotient one ulp off shows
    pw = torch.pow(2.0, torch.arange(-10, 10, dtype=torch.float32))
    key[0, 0, :20] = (pw * scale).to(torch.bfloat16)
    grid = torch.arange(0, 256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    grid = grid[torch.isfinite(grid) & (grid > 0)].sort().values
    mids = ((grid[1:] + grid[:-1]) / 2)[:d]
    value[1, 1, : mids.numel()] = (mids * scale).to(torch.bfloat16)
    slots = torch.randperm(toks // bs, generator=g).repeat_interleave(bs) * bs + torch.arange(toks) % bs
    kref = L.tokens_to_key_cache((key.float() / scale).clamp(-448, 448).to(torch.float8_e4m3fn).view(toks // bs, bs, h, d))
    vref = L.tokens_to_value_cache((value.float() / scale).clamp(-448, 448).to(torch.float8_e4m3fn).view(toks // bs, bs, h, d))
    order = (slots.view(-1, bs)[:, 0] // bs)
    kc = torch.zeros(kref.shape, dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
    vc = torch.zeros(vref.shape, dtype=torch.uint8, device=cuda).view(torch.float8_e4m3fn)
    s_dev = scale.to(cuda)
    T.kv_cache_write(key.to(cuda), value.to(cuda), kc, vc, slots.to(cuda), s_dev, s_dev)
    torch.cuda.synchronize()
    assert torch.equal(kc.cpu().view(torch.uint8)[order], kref.view(torch.uint8))
    assert torch.equal(vc.cpu().view(torch.uint8)[order], vref.view(torch.uint8))
