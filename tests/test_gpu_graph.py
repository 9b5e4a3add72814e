"""Every entry point under HIP graph capture: the library launches kernels only (no memset nodes, no
host round trips, no allocation), so a captured sequence must replay to the eager result.  Each graph is
replayed three times on fresh inputs, with eager work and synchronisations between the replays, and every
replay is compared bit for bit with the eager call on the same inputs."""
import pytest
import torch

from cosmos_rl_amd import ops

pytestmark = pytest.mark.gpu


def _replay_matches_eager(dev, make_inputs, fn, seeds=(11, 12, 13)):
    """fn(*inputs) -> tuple of tensors.  Captures fn on static inputs, then for every seed copies fresh
    inputs in, replays, and compares with an eager fn on clones of the same inputs."""
    static_in = [t.clone() for t in make_inputs(seeds[0] - 1)]
    for _ in range(2):                      # warm-up outside the capture: one-time host setup happens here
        fn(*static_in)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            static_out = fn(*static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for seed in seeds:
        fresh = make_inputs(seed)
        for s, f in zip(static_in, fresh):
            s.copy_(f)
        g.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in static_out]
        want = fn(*[f.clone() for f in fresh])          # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert a.dtype == b.dtype and a.shape == b.shape
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), (seed, a.dtype, tuple(a.shape))


def _bf16(dev, seed, *shape, std=1.0):
    g = torch.Generator(device=dev).manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=dev) * std).to(torch.bfloat16)


def test_graph_weight_quantisers(dev):
    def inputs(seed):
        return [_bf16(dev, seed, 512, 896, std=0.02), _bf16(dev, seed + 100, 300, 256, std=0.02), _bf16(dev, seed + 200, 1024, std=0.02)]

    def fn(a, b, c):
        qa, sa = ops.quant_rowwise(a)
        outs, scales = ops.quant_tensorwise_multi([a, b, c])
        qb, sb = ops.per_block_cast_to_fp8(a)
        qg, sg = ops.groupwise_activation_quant(a)
        q4, s4 = ops.quant_mxfp4(a)
        back = ops.weight_dequant(qb, sb)
        return (qa, sa, *outs, scales, qb, sb, qg, sg, q4, s4, back)

    _replay_matches_eager(dev, inputs, fn)


def test_graph_batch_quantisers_without_allocation(dev):
    """The table-driven rowwise quantiser and the tensorwise entry point whose amax slots live inside the library,
    captured with caller-owned outputs: nothing inside the captured region allocates."""
    shapes = [(512, 896), (300, 256), (64, 3584), (16, 18944)]
    qs = [torch.empty(sh, dtype=torch.float8_e4m3fn, device=dev) for sh in shapes]
    ss = [torch.empty(sh[0], 1, dtype=torch.float32, device=dev) for sh in shapes]
    qt = [torch.empty(sh, dtype=torch.float8_e4m3fn, device=dev) for sh in shapes]
    st = torch.empty(len(shapes), dtype=torch.float32, device=dev)

    def inputs(seed):
        return [_bf16(dev, seed + 10 * i, *sh, std=0.02 * (i + 1)) for i, sh in enumerate(shapes)]

    def fn(*ws):
        ops.quant_rowwise_multi_into(list(ws), qs, ss)
        ops.quant_tensorwise_multi_static(list(ws), qt, st)
        return (*qs, *ss, *qt, st)

    _replay_matches_eager(dev, inputs, fn)
    # and the captured results are the per-tensor ones
    ws = inputs(13)
    for w, q, sc in zip(ws, qs, ss):
        q1, s1 = ops.quant_rowwise(w)
        assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(sc, s1)


def test_graph_tensorwise_read_once_launch(dev):
    """A tensor large enough for the launch that keeps it on the chip between the passes (its workgroups meet at a
    counter in device memory, cleared by the fill kernel in front of it), captured together with a small one."""
    shapes = [(18944, 3584), (300, 256)]
    qt = [torch.empty(sh, dtype=torch.float8_e4m3fn, device=dev) for sh in shapes]
    st = torch.empty(len(shapes), dtype=torch.float32, device=dev)

    def inputs(seed):
        return [_bf16(dev, seed + 10 * i, *sh, std=0.02 * (i + 1)) for i, sh in enumerate(shapes)]

    def fn(*ws):
        ops.quant_tensorwise_multi_static(list(ws), qt, st)
        return (*qt, st)

    _replay_matches_eager(dev, inputs, fn)


@pytest.mark.parametrize("M,N,K", [(1, 2048, 3584), (64, 2048, 3584), (48, 1024, 7168), (1024, 2048, 3584), (2304, 8448, 256), (2048, 8704, 512)])
def test_graph_fp8_linear(dev, M, N, K):
    """single-token and 64-token kernels, the split-K pair of launches, 256x256 tiles, the head + tail pair, and the
    walking kernel with a last round taken as quarter tiles"""
    w = _bf16(dev, 5, N, K, std=0.02)
    qw, sw = ops.quant_rowwise(w)

    def inputs(seed):
        return [_bf16(dev, seed, M, K)]

    def fn(x):
        return (ops.fp8_linear(x, qw.t(), sw), ops.fp8_linear(x, qw.t(), sw, out_dtype=torch.float32))

    _replay_matches_eager(dev, inputs, fn)


def test_graph_block_gemm_256x256_tiles(dev):
    """1x128 activation quantiser + the block-scaled GEMM on 256 x 256 tiles with its last tile-column as a second
    launch (272 tiles), and a K that is a multiple of 16 only through the rowwise linear's masked last step."""
    M, N, K = 4096, 4352, 2048
    qw, sw = ops.per_block_cast_to_fp8(_bf16(dev, 6, N, K, std=0.02))
    w2 = _bf16(dev, 7, 512, 1200, std=0.02)
    qw2, sw2 = ops.quant_rowwise(w2)

    def inputs(seed):
        return [_bf16(dev, seed, M, K), _bf16(dev, seed + 100, 100, 1200)]

    def fn(x, x2):
        qx, sx = ops.groupwise_activation_quant(x)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
        ops.gemm_fp8_fp8_bf16_nt((qx, sx), (qw, sw), out)
        return (out, ops.fp8_linear(x2, qw2.t(), sw2))

    _replay_matches_eager(dev, inputs, fn)


def test_graph_moe_chain(dev):
    from cosmos_rl_amd import _lib
    from cosmos_rl_amd.policy.kernel.moe.moe import combine_expert_outputs, route_tokens
    from cosmos_rl_amd.policy.kernel.moe.indices import permute_tokens
    T, K, E, H, I = 256, 4, 8, 256, 128
    gen = torch.Generator(device=dev).manual_seed(3)
    wgu, wd = _bf16(dev, 1, E, 2 * I, H, std=0.05), _bf16(dev, 2, E, H, I, std=0.05)
    qgu, sgu = ops.per_block_cast_to_fp8(wgu)
    qd, sd = ops.per_block_cast_to_fp8(wd)
    qgi, sgi = ops.interleave_gate_up((qgu[:, :I], sgu[:, :I // 128]), (qgu[:, I:], sgu[:, I // 128:]))
    rows_cap = T * K + E * 128

    def inputs(seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        logits = torch.rand(T, E, generator=g, device=dev)
        top = torch.topk(logits, K, dim=1)
        return [_bf16(dev, seed, T, H), top.indices.to(torch.int32), top.values.to(torch.bfloat16)]

    def fn(x, idx, wts):
        r = route_tokens(idx, None, E, 128, max_rows=rows_cap)
        contig = permute_tokens(x, r.row_tokens)
        m_idx = ops.create_indices_from_offsets_nosync(r.m_offsets, rows_cap)
        m_idx = torch.where((r.row_tokens >= 0) & (m_idx < E), m_idx, torch.full_like(m_idx, -1))
        qx, sx = ops.groupwise_activation_quant(contig)
        gu = torch.zeros(rows_cap, 2 * I, dtype=torch.bfloat16, device=dev)
        ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qx, sx), (qgu, sgu), gu, m_idx)
        qh, sh = ops.swiglu_quant(gu[:, :I], gu[:, I:])
        qh_e, sh_e = ops.grouped_gemm_swiglu_quant((qx, sx), (qgi, sgi), m_idx)   # the same as the GEMM's epilogue
        keep = (m_idx >= 0)[:, None]
        qh_e = torch.where(keep, qh_e.view(torch.uint8), torch.zeros_like(qh_e.view(torch.uint8)))
        sh_e = torch.where(keep, sh_e, torch.zeros_like(sh_e))
        dn = torch.zeros(rows_cap, H, dtype=torch.bfloat16, device=dev)
        ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((qh, sh), (qd, sd), dn, m_idx)
        y = combine_expert_outputs(dn, r, wts)
        return (r.row_tokens, r.row_map, m_idx, qx, gu, qh, dn, y, qh_e, sh_e)

    _replay_matches_eager(dev, inputs, fn)
