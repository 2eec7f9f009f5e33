"""The grouped int8 GEMM operators on the GPU against the CPU oracle.

Bars: int32 accumulators bit-exact; bf16 / fp16 outputs of the down projection bit-exact (same fp32 operation order,
nearest-even casts); SwiGLU-quant int8 within +-1 LSB and scales within 1e-2 relative (in practice ~1e-6: only the
device's expf and divide can differ from the host's).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(rng, M, K, N, E, mode="ragged"):
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)  # K-contiguous storage
    if mode == "ragged":
        cuts = np.sort(rng.integers(0, M + 1, E - 1)) if E > 1 else np.array([], np.int64)
        cumsum = np.concatenate([cuts, [M]]).astype(np.int64)
    elif mode == "even":
        cumsum = ((np.arange(1, E + 1) * M) // E).astype(np.int64)
    elif mode == "sparse":  # most groups empty
        sizes = np.zeros(E, np.int64)
        hot = rng.choice(E, max(1, E // 8), replace=False)
        sizes[hot] = rng.multinomial(M, np.ones(len(hot)) / len(hot))
        cumsum = np.cumsum(sizes)
    return x, wt, cumsum


def _weight_views(wt, dev, layout):
    """[E, K, N] view for the operator: transposed view of K-contiguous storage, or a contiguous ND tensor."""
    w_dev = torch.from_numpy(wt).to(dev)
    if layout == "kmajor":
        return w_dev.transpose(1, 2)
    return w_dev.transpose(1, 2).contiguous()


INT32_CASES = [  # M, K, N, E, mode, layout
    (1, 16, 8, 1, "even", "kmajor"),
    (37, 128, 24, 4, "ragged", "kmajor"),
    (37, 128, 2, 4, "ragged", "kmajor"),         # one expert's weights are shorter than a kilobyte: byte-wise loader
    (64, 384, 2, 3, "even", "kmajor"),
    (37, 128, 6, 4, "ragged", "kmajor"),
    (37, 128, 8, 4, "ragged", "kmajor"),         # exactly one kilobyte per expert: the ring kernel
    (96, 256, 300, 7, "ragged", "kmajor"),
    (512, 1024, 512, 8, "even", "kmajor"),       # tile 96
    (512, 4096, 256, 128, "ragged", "kmajor"),   # decode-like: tile 32, many groups
    (700, 512, 520, 3, "ragged", "kmajor"),      # tile 256, N not a multiple of the tile
    (1500, 384, 256, 10, "ragged", "kmajor"),    # tile 192 + partial tiles
    (2048, 2048, 256, 16, "even", "kmajor"),     # tile 192, exact 128-row groups
    (300, 200, 64, 4, "ragged", "kmajor"),       # K not a multiple of 16: byte-wise loader
    (300, 208, 72, 4, "ragged", "nd"),           # row-major [E,K,N] weight: byte-wise loader
    (100, 7168, 64, 2, "even", "kmajor"),        # |acc| beyond 2^24
    (640, 256, 256, 64, "sparse", "kmajor"),
    # row-major [E, K, N] weights (the reference's plain ND layout) on the fast kernel: K % 128 == 0, N % 16 == 0
    (37, 128, 16, 4, "ragged", "nd"),
    (512, 1024, 512, 8, "even", "nd"),
    (700, 512, 528, 3, "ragged", "nd"),          # tile 256; 528 = 2 * 256 + 16 channels: the last tile holds one chunk
    (1500, 384, 256, 10, "ragged", "nd"),
    (512, 4096, 256, 128, "ragged", "nd"),       # decode-like
    (640, 256, 272, 64, "sparse", "nd"),
]


@pytest.mark.parametrize("M,K,N,E,mode,layout", INT32_CASES)
def test_int32_accumulators_bit_exact(aclnn, oracle, dev, M, K, N, E, mode, layout):
    rng = np.random.default_rng(M * 3 + K + N)
    x, wt, cumsum = _problem(rng, M, K, N, E, mode)
    ref = oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True)
    xd = torch.from_numpy(x).to(dev)
    wv = _weight_views(wt, dev, layout)
    for list_type, dtype in ((0, torch.int64), (1, torch.int64), (0, torch.int32)):
        gl = cumsum if list_type == 0 else np.diff(np.concatenate([[0], cumsum]))
        out = torch.full((M, N), -7, dtype=torch.int32, device=dev)
        aclnn.grouped_matmul_v4([xd], [wv], group_list=torch.from_numpy(gl).to(dev).to(dtype), split_item=3, group_type=0,
                                group_list_type=list_type, out=[out])
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), ref)


def test_rows_beyond_last_group_untouched(aclnn, oracle, dev):
    rng = np.random.default_rng(4)
    x, wt, _ = _problem(rng, 200, 128, 64, 3, "even")
    cumsum = np.array([50, 50, 120], np.int64)
    out = torch.full((200, 64), -7, dtype=torch.int32, device=dev)
    aclnn.grouped_matmul_v4([torch.from_numpy(x).to(dev)], [_weight_views(wt, dev, "kmajor")],
                            group_list=torch.from_numpy(cumsum).to(dev), split_item=3, group_type=0, out=[out])
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    ref = oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True)
    assert np.array_equal(got[:120], ref[:120]) and (got[120:] == -7).all()


@pytest.mark.parametrize("kind,values", [
    ("cumsum", [300, 0, 300, 0, 300]),          # groups 0, 2 and 4 each claim every row: three times the tiles of a sane list
    ("cumsum", [120, 50, 400, -7, 90]),         # not monotonic, beyond M, negative
    ("count", [300, 300, 300, 300, 300]),       # counts add up to five times M
    ("count", [-5, 400, 10, 0, 2000000000]),
])
def test_malformed_group_lists_stay_in_bounds(aclnn, dev, kind, values):
    """A list that is not a cumsum / count list of M rows gives unspecified rows, but never an access outside the
    tensors: boundaries are clamped into [0, M] and the tile table is cut at the size planned for a well-formed list."""
    rng = np.random.default_rng(9)
    M, K, N, E = 300, 128, 64, 5
    x, wt, _ = _problem(rng, M, K, N, E, "even")
    guard = torch.full((M + 64, N), -7, dtype=torch.int32, device=dev)
    aclnn.grouped_matmul_v4([torch.from_numpy(x).to(dev)], [_weight_views(wt, dev, "kmajor")],
                            group_list=torch.tensor(values, dtype=torch.int64, device=dev), split_item=3, group_type=0,
                            group_list_type=0 if kind == "cumsum" else 1, out=[guard[:M]])
    torch.cuda.synchronize()
    assert (guard[M:] == -7).all()


DEQUANT_CASES = [(64, 256, 128, 4, "f32", torch.bfloat16), (64, 256, 128, 4, "bf16", torch.bfloat16),
                 (64, 256, 128, 4, "f32", torch.float16), (512, 1024, 1024, 8, "f32", torch.bfloat16),
                 (333, 1536, 520, 16, "f32", torch.bfloat16)]


@pytest.mark.parametrize("M,K,N,E,scale_dtype,out_dtype", DEQUANT_CASES)
def test_down_projection_epilogue(aclnn, oracle, dev, M, K, N, E, scale_dtype, out_dtype):
    rng = np.random.default_rng(M + N)
    x, wt, cumsum = _problem(rng, M, K, N, E)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    per_token = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    scale_t = torch.from_numpy(scale).to(dev)
    if scale_dtype == "bf16":
        scale_t = scale_t.to(torch.bfloat16)
        scale_arg, sd = scale_t.view(torch.int16).cpu().numpy().view(np.uint16), oracle.DT_BF16
    else:
        scale_arg, sd = scale, oracle.DT_F32
    od = oracle.DT_BF16 if out_dtype == torch.bfloat16 else oracle.DT_F16
    ref = oracle.grouped_matmul_dequant(x, wt, scale_arg, per_token, cumsum, w_trans=True, scale_dtype=sd, out_dtype=od)
    for layout in ("kmajor", "nd"):       # K-contiguous storage behind a transposed view, and row-major [E, K, N]
        out = aclnn.grouped_matmul_v4([torch.from_numpy(x).to(dev)], [_weight_views(wt, dev, layout)], scale=[scale_t],
                                      per_token_scale=[torch.from_numpy(per_token).to(dev)],
                                      group_list=torch.from_numpy(cumsum).to(dev), split_item=3, group_type=0,
                                      output_dtype=out_dtype)[0]
        torch.cuda.synchronize()
        assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), ref), layout


SWIGLU_CASES = [  # M, K, N, E, mode, layout, scale dtype
    (16, 256, 512, 4, "even", "kmajor", "f32"),       # reference tiling UT shape
    (192, 2048, 2048, 4, "ragged", "kmajor", "f32"),  # reference op_api UT shape
    (512, 1024, 2048, 8, "ragged", "kmajor", "f32"),  # small config
    (512, 4096, 3072, 128, "ragged", "kmajor", "f32"),  # decode config shape
    (300, 512, 208, 5, "ragged", "kmajor", "bf16"),   # N/2 not a multiple of the tile
    (300, 512, 208, 5, "ragged", "kmajor", "f16"),
    (100, 200, 96, 3, "ragged", "nd", "f32"),
    (512, 1024, 2048, 8, "ragged", "nd", "f32"),      # row-major weights on the fast kernel
    (300, 512, 224, 5, "ragged", "nd", "bf16"),       # N/2 = 112 = 7 chunks: both halves of the tile are clamped
    (512, 4096, 3072, 128, "ragged", "nd", "f32"),
]


@pytest.mark.parametrize("M,K,N,E,mode,layout,sdt", SWIGLU_CASES)
def test_swiglu_quant(aclnn, oracle, dev, M, K, N, E, mode, layout, sdt):
    rng = np.random.default_rng(M + K + N)
    x, wt, cumsum = _problem(rng, M, K, N, E, mode)
    used = int(M * 0.9)
    cumsum = np.minimum(cumsum, used)  # trailing rows belong to no group and must stay untouched
    w_scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    x_scale = rng.uniform(5e-3, 5e-2, M).astype(np.float32)
    ws_t = torch.from_numpy(w_scale).to(dev)
    if sdt == "bf16":
        ws_t = ws_t.to(torch.bfloat16)
        ws_arg, code = ws_t.view(torch.int16).cpu().numpy().view(np.uint16), oracle.DT_BF16
    elif sdt == "f16":
        ws_t = ws_t.to(torch.float16)
        ws_arg, code = ws_t.view(torch.int16).cpu().numpy().view(np.uint16), oracle.DT_F16
    else:
        ws_arg, code = w_scale, oracle.DT_F32
    y_ref, ys_ref = oracle.grouped_matmul_swiglu_quant(x, wt, ws_arg, x_scale, cumsum, w_trans=True, w_scale_dtype=code)
    y = torch.full((M, N // 2), 55, dtype=torch.int8, device=dev)
    ys = torch.full((M,), -3.0, dtype=torch.float32, device=dev)
    aclnn.grouped_matmul_swiglu_quant(torch.from_numpy(x).to(dev), _weight_views(wt, dev, layout),
                                      torch.from_numpy(cumsum).to(dev), ws_t, torch.from_numpy(x_scale).to(dev),
                                      out=(y, ys))
    torch.cuda.synchronize()
    y, ys = y.cpu().numpy(), ys.cpu().numpy()
    last = int(cumsum[-1])
    diff = np.abs(y[:last].astype(np.int32) - y_ref[:last].astype(np.int32))
    assert diff.max() <= 1, "int8 output differs by %d LSB" % diff.max()
    assert (diff != 0).mean() < 1e-3
    np.testing.assert_allclose(ys[:last], ys_ref[:last], rtol=1e-2)
    np.testing.assert_allclose(ys[:last], ys_ref[:last], rtol=1e-5)  # observed: only expf / divide rounding differs
    assert (y[last:] == 55).all() and (ys[last:] == -3.0).all()


def test_swiglu_empty_group_list_is_noop(aclnn, dev):
    x = torch.zeros((4, 32), dtype=torch.int8, device=dev)
    w = torch.zeros((2, 64, 32), dtype=torch.int8, device=dev).transpose(1, 2)
    gl = torch.empty((0,), dtype=torch.int64, device=dev)
    y, ys = aclnn.grouped_matmul_swiglu_quant(x, w, gl, torch.ones((2, 64), device=dev), torch.ones((4,), device=dev))
    torch.cuda.synchronize()
    assert y.shape == (4, 32)


@pytest.mark.parametrize("hint", [[], [16], [96], [4096]])
def test_v5_tuning_hint_changes_tiling_not_results(aclnn, oracle, dev, hint):
    """aclnnGroupedMatmulV5's tuningConfig picks another tile height; the int32 accumulators stay bit-exact."""
    rng = np.random.default_rng(55)
    M, K, N, E = 900, 512, 320, 6
    x, wt, cumsum = _problem(rng, M, K, N, E, "ragged")
    ref = oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True)
    out = aclnn.grouped_matmul_v5([torch.from_numpy(x).to(dev)], [_weight_views(wt, dev, "kmajor")], tuning_config=hint,
                                  group_list=torch.from_numpy(cumsum).to(dev), split_item=3, group_type=0,
                                  group_list_type=0, act_type=0, output_dtype=torch.int32)[0]
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), ref)


# ------------------------------------------------------------------------------------------------ sparse group lists
@pytest.mark.parametrize("M,K,N,E,order", [(300, 256, 256, 16, "ascending"), (640, 512, 520, 64, "ascending"),
                                          (200, 128, 128, 8, "shuffled"), (96, 128, 72, 4, "all")])
def test_sparse_group_list(aclnn, oracle, dev, M, K, N, E, order):
    """groupListType 2: [E, 2] pairs (expert id, rows) in row order, ended by the first pair without rows
    (gmm/grouped_matmul/op_kernel/grouped_matmul.h:288-345).  The oracle sees the same problem as a dense count list over
    the weights picked by the pairs."""
    rng = np.random.default_rng(M + E)
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    used = E if order == "all" else max(1, E // 3)
    keys = np.sort(rng.choice(E, used, replace=False))
    if order == "shuffled":
        rng.shuffle(keys)
    covered = M - 11                                              # the last rows belong to no pair
    counts = rng.multinomial(covered - used, np.ones(used) / used) + 1
    pairs = np.zeros((E, 2), np.int64)
    pairs[:used, 0], pairs[:used, 1] = keys, counts
    pairs[used:, 0] = rng.integers(0, E, E - used)                # ids behind the end marker are never read as groups
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    xd, wv = torch.from_numpy(x).to(dev), torch.from_numpy(wt).to(dev).transpose(1, 2)
    out = torch.full((M, N), -7, dtype=torch.int32, device=dev)
    aclnn.grouped_matmul_v4([xd], [wv], group_list=torch.from_numpy(pairs).to(dev), split_item=3, group_type=0,
                            group_list_type=2, out=[out])
    y = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    aclnn.grouped_matmul_v4([xd], [wv], scale=[torch.from_numpy(scale).to(dev)], per_token_scale=[torch.from_numpy(pt).to(dev)],
                            group_list=torch.from_numpy(pairs).to(dev), split_item=3, group_type=0, group_list_type=2, out=[y])
    torch.cuda.synchronize()
    ref = oracle.grouped_matmul_i32(x, wt[keys], counts.astype(np.int64), list_type=1, w_trans=True)
    got = out.cpu().numpy()
    assert np.array_equal(got[:covered], ref[:covered])
    assert (got[covered:] == -7).all()
    ref_y = oracle.grouped_matmul_dequant(x, wt[keys], scale[keys], pt, counts.astype(np.int64), list_type=1, w_trans=True,
                                          out_dtype=oracle.DT_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16)[:covered], ref_y[:covered])


def test_sparse_list_from_routing_v3(aclnn, oracle, dev):
    """MoeInitRoutingV3's key/value count output is the sparse list GroupedMatmulV4 takes."""
    rng = np.random.default_rng(3)
    T, K, E, H, N = 96, 2, 32, 128, 64
    x = rng.integers(-127, 128, (T, H)).astype(np.int8)
    idx = rng.choice(E // 4, (T, K)).astype(np.int32) * 4          # only every fourth expert is used
    wt = rng.integers(-127, 128, (E, N, H)).astype(np.int8)
    ex, _, pairs, _ = aclnn.moe_init_routing_v3(torch.from_numpy(x).to(dev), torch.from_numpy(idx).to(dev), None,
                                                expert_num=E, expert_tokens_num_type=2)
    out = torch.zeros((T * K, N), dtype=torch.int32, device=dev)
    aclnn.grouped_matmul_v4([ex], [torch.from_numpy(wt).to(dev).transpose(1, 2)], group_list=pairs, split_item=3,
                            group_type=0, group_list_type=2, out=[out])
    torch.cuda.synchronize()
    ex_r, _, cnt_r, _ = oracle.moe_init_routing_v3(x, idx, None, E, None, 1, 1)
    ref = oracle.grouped_matmul_i32(ex_r, wt, cnt_r, list_type=1, w_trans=True)
    assert np.array_equal(out.cpu().numpy(), ref)


# ------------------------------------------------------------------------------------------------ FRACTAL_NZ weights
def _to_nz(w_ekn):
    """[E, K, N] -> the blocked layout [E, N/32, K/16, 16, 32]: element (k, n) at [n / 32][k / 16][k % 16][n % 32]."""
    E, K, N = w_ekn.shape
    return np.ascontiguousarray(w_ekn.reshape(E, K // 16, 16, N // 32, 32).transpose(0, 3, 1, 2, 4))


NZ_CASES = [  # M, K, N, E, mode, how
    (37, 128, 64, 4, "ragged", "nz5d"),            # N/2 = 32: one channel block per half
    (96, 256, 320, 7, "ragged", "entry5d"),        # partial n-tile
    (512, 1024, 512, 8, "even", "entry3d"),
    (512, 4096, 3072, 128, "ragged", "nz5d"),      # decode shape
    (700, 512, 576, 3, "ragged", "nz5d"),          # 256-row tiles
    (300, 208, 128, 4, "ragged", "nz5d"),          # K not a multiple of 128: byte-wise kernel
    (2048, 2048, 512, 16, "even", "entry5d"),
]


@pytest.mark.parametrize("M,K,N,E,mode,how", NZ_CASES)
def test_swiglu_quant_nz_weight_equals_nd_weight(aclnn, oracle, dev, M, K, N, E, mode, how):
    """The blocked weight layout gives exactly what the same weights give as an ND tensor (same arithmetic, other
    addressing), and that stays within the operator's bars against the oracle."""
    rng = np.random.default_rng(M + K + N)
    x, wt, cumsum = _problem(rng, M, K, N, E, mode)            # wt: [E, N, K] storage
    w_ekn = np.ascontiguousarray(wt.transpose(0, 2, 1))
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    xs = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    q_nd, s_nd = aclnn.grouped_matmul_swiglu_quant(t(x), t(wt).transpose(1, 2), t(cumsum), t(scale), t(xs))
    q_nz, s_nz = aclnn.grouped_matmul_swiglu_quant(t(x), None, t(cumsum), t(scale), t(xs), weight_nz=(t(_to_nz(w_ekn)), how))
    torch.cuda.synchronize()
    rows = int(cumsum[-1])
    assert torch.equal(q_nd[:rows], q_nz[:rows]) and torch.equal(s_nd[:rows], s_nz[:rows])
    ref_q, ref_s = oracle.grouped_matmul_swiglu_quant(x, wt, scale, xs, cumsum, w_trans=True)
    assert np.abs(q_nz.cpu().numpy()[:rows].astype(np.int32) - ref_q[:rows].astype(np.int32)).max() <= 1
    np.testing.assert_allclose(s_nz.cpu().numpy()[:rows], ref_s[:rows], rtol=1e-2)


@pytest.mark.parametrize("M,K,N,E,mode,how", [(37, 128, 64, 4, "ragged", "nz5d"), (96, 256, 320, 7, "ragged", "entry5d"),
                                              (512, 1024, 512, 8, "even", "entry3d"), (700, 512, 544, 3, "ragged", "nz5d"),
                                              (300, 208, 96, 4, "ragged", "entry3d"), (512, 1536, 4096, 128, "ragged", "nz5d")])
def test_grouped_matmul_nz_weight(aclnn, oracle, dev, M, K, N, E, mode, how):
    """int32 accumulators and the bf16 down-projection output with a blocked weight: bit-exact against the oracle."""
    rng = np.random.default_rng(M + K + N + 1)
    x, wt, cumsum = _problem(rng, M, K, N, E, mode)
    w_nz = torch.from_numpy(_to_nz(np.ascontiguousarray(wt.transpose(0, 2, 1)))).to(dev)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    acc = aclnn.grouped_matmul_v4([t(x)], None, group_list=t(cumsum), split_item=3, group_type=0, weight_nz=(w_nz, how))[0]
    y = aclnn.grouped_matmul_v4([t(x)], None, scale=[t(scale)], per_token_scale=[t(pt)], group_list=t(cumsum), split_item=3,
                                group_type=0, output_dtype=torch.bfloat16, weight_nz=(w_nz, how), tuning_config=[M // E])[0]
    torch.cuda.synchronize()
    rows = int(cumsum[-1])
    assert np.array_equal(acc.cpu().numpy()[:rows], oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True)[:rows])
    ref = oracle.grouped_matmul_dequant(x, wt, scale, pt, cumsum, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16)[:rows], ref[:rows])


# ------------------------------------------------------------------------------------------------ every instantiation
@pytest.mark.parametrize("layout", ["kmajor", "nz", "nd"])
@pytest.mark.parametrize("tile_m", [32, 64, 96, 128, 160, 192, 256])
def test_every_tile_height_and_layout(aclnn, oracle, dev, monkeypatch, tile_m, layout):
    """The fast kernel is compiled once per (tile height, weight layout, epilogue).  The planner picks the height from the
    group sizes, so the hand-picked shapes reach only some of the 63; here the height is forced and one ragged problem
    (groups of 0 to ~400 rows, a partial n-tile) runs through all three epilogues of each one: int32 and bf16 bit-exact,
    SwiGLU-quant to +-1 LSB."""
    monkeypatch.setenv("OPAPI_GEMM_TILE_M", str(tile_m))
    rng = np.random.default_rng(77)
    M, K, N, E = 900, 384, 320, 6
    x, wt, cumsum = _problem(rng, M, K, N, E, "ragged")
    cumsum[1] = cumsum[0]                                        # one empty group
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    if layout == "nz":
        w_nz = t(_to_nz(np.ascontiguousarray(wt.transpose(0, 2, 1))))
        wkw, wv, wsw = dict(weight_nz=(w_nz, "nz5d")), None, dict(weight_nz=(w_nz, "nz5d"))
    else:
        wkw, wv, wsw = {}, [_weight_views(wt, dev, layout)], {}
    acc = aclnn.grouped_matmul_v4([t(x)], wv, group_list=t(cumsum), split_item=3, group_type=0, **wkw)[0]
    y = aclnn.grouped_matmul_v4([t(x)], wv, scale=[t(scale)], per_token_scale=[t(pt)], group_list=t(cumsum), split_item=3,
                                group_type=0, output_dtype=torch.bfloat16, **wkw)[0]
    q, qs = aclnn.grouped_matmul_swiglu_quant(t(x), wv[0] if wv else None, t(cumsum), t(scale), t(pt), **wsw)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True))
    ref = oracle.grouped_matmul_dequant(x, wt, scale, pt, cumsum, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), ref)
    q_ref, qs_ref = oracle.grouped_matmul_swiglu_quant(x, wt, scale, pt, cumsum, w_trans=True)
    diff = np.abs(q.cpu().numpy().astype(np.int32) - q_ref.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
    np.testing.assert_allclose(qs.cpu().numpy(), qs_ref, rtol=1e-5)


@pytest.mark.parametrize("K", [128, 256, 640])
@pytest.mark.parametrize("tile_m", [32, 64, 96, 128, 160, 192, 256])
def test_many_tiles_per_workgroup_every_height(aclnn, oracle, dev, monkeypatch, tile_m, K):
    """Every workgroup of the persistent kernel walks several tiles here, and a tile is one, two or five k-steps long --
    shorter than the LDS ring is deep -- so the issue cursors run a tile or more ahead of the MFMAs, cross tile
    boundaries at different times (the 192-row kernel keeps one cursor per operand) and drain at the end of the walk.
    The forced-height test above has fewer tiles than workgroups and never gets there.  int32 output, bit-exact."""
    monkeypatch.setenv("OPAPI_GEMM_TILE_M", str(tile_m))
    rng = np.random.default_rng(1000 * tile_m + K)
    E, N = 48, 256 * 8 + 64
    sizes = rng.integers(0, 230, E)
    sizes[5] = 0
    sizes[17] = 257                      # one group past the tallest tile
    cumsum = np.cumsum(sizes).astype(np.int64)
    M = int(cumsum[-1])
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    t = lambda a: torch.from_numpy(a).to(dev)
    acc = aclnn.grouped_matmul_v4([t(x)], [_weight_views(wt, dev, "kmajor")], group_list=t(cumsum), split_item=3, group_type=0)[0]
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True))


@pytest.mark.parametrize("layout", ["nz", "nd"])
@pytest.mark.parametrize("tile_m", [128, 192, 256])
def test_many_tiles_per_workgroup_other_layouts(aclnn, oracle, dev, monkeypatch, tile_m, layout):
    """The same walk with the blocked and the row-major weight layouts (bf16 output of the down projection as well)."""
    monkeypatch.setenv("OPAPI_GEMM_TILE_M", str(tile_m))
    rng = np.random.default_rng(31 * tile_m + len(layout))
    E, N, K = 40, 256 * 8 + 64, 256
    sizes = rng.integers(0, 230, E)
    cumsum = np.cumsum(sizes).astype(np.int64)
    M = int(cumsum[-1])
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    if layout == "nz":
        wkw, wv = dict(weight_nz=(t(_to_nz(np.ascontiguousarray(wt.transpose(0, 2, 1)))), "nz5d")), None
    else:
        wkw, wv = {}, [_weight_views(wt, dev, layout)]
    acc = aclnn.grouped_matmul_v4([t(x)], wv, group_list=t(cumsum), split_item=3, group_type=0, **wkw)[0]
    y = aclnn.grouped_matmul_v4([t(x)], wv, scale=[t(scale)], per_token_scale=[t(pt)], group_list=t(cumsum), split_item=3,
                                group_type=0, output_dtype=torch.bfloat16, **wkw)[0]
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True))
    ref = oracle.grouped_matmul_dequant(x, wt, scale, pt, cumsum, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), ref)


@pytest.mark.parametrize("K", [1024, 1152])
@pytest.mark.parametrize("tile_m", [32, 64, 96, 128, 160, 192, 256])
def test_pulled_tiles_under_skew_every_height(aclnn, oracle, dev, monkeypatch, tile_m, K):
    """Tiles of eight k-steps and more are drawn from the tile counters (forced on here for the two smallest heights as
    well).  A skewed list -- two groups of many m-tiles, a few of a few hundred rows, many of a handful, some empty,
    sizes either side of the small-tile limit of 64 rows and of each tile height -- fills both runs of the m-tile
    table, gives every workgroup several tiles, and ends with workgroups drawing from other XCDs' shares.  K = 1024 is
    the shortest tile that is pulled (the issue side reaches the tile after next exactly when it has been drawn).
    int32 output bit-exact, and the down-projection epilogue on the same list."""
    monkeypatch.setenv("OPAPI_GEMM_TILE_M", str(tile_m))
    monkeypatch.setenv("OPAPI_GEMM_PULL", "1")
    rng = np.random.default_rng(7 * tile_m + K)
    N = 256 * 16 + 64
    sizes = [1500, 3, 700, 0, 40, 300, 1, 65, 64, 513, 0, 63, tile_m, tile_m + 1, max(tile_m - 1, 1), 2 * tile_m]
    sizes += [int(v) for v in rng.integers(1, 24, 30)]
    sizes = np.array(sizes)
    E = len(sizes)
    cumsum = np.cumsum(sizes).astype(np.int64)
    M = int(cumsum[-1])
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    wv = [_weight_views(wt, dev, "kmajor")]
    acc = aclnn.grouped_matmul_v4([t(x)], wv, group_list=t(cumsum), split_item=3, group_type=0)[0]
    y = aclnn.grouped_matmul_v4([t(x)], wv, scale=[t(scale)], per_token_scale=[t(pt)], group_list=t(sizes.astype(np.int64)),
                                split_item=3, group_type=0, group_list_type=1, output_dtype=torch.bfloat16)[0]
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), oracle.grouped_matmul_i32(x, wt, cumsum, w_trans=True))
    ref = oracle.grouped_matmul_dequant(x, wt, scale, pt, cumsum, w_trans=True, out_dtype=oracle.DT_BF16)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), ref)
    # the same launch with fixed shares gives the same bits
    monkeypatch.setenv("OPAPI_GEMM_PULL", "0")
    acc_fixed = aclnn.grouped_matmul_v4([t(x)], wv, group_list=t(cumsum), split_item=3, group_type=0)[0]
    torch.cuda.synchronize()
    assert torch.equal(acc, acc_fixed)


def test_pulled_tiles_swiglu_skewed(aclnn, oracle, dev, monkeypatch):
    """The SwiGLU epilogue on a skewed list with pulled tiles (the requantisation reads rows written by tiles that ran
    in no fixed order)."""
    monkeypatch.setenv("OPAPI_GEMM_PULL", "1")
    rng = np.random.default_rng(99)
    K, N = 1024, 2048
    sizes = np.array([900, 2, 0, 300, 17, 64, 65, 1, 5, 130, 40, 0, 7] + [int(v) for v in rng.integers(1, 12, 20)])
    E = len(sizes)
    cumsum = np.cumsum(sizes).astype(np.int64)
    M = int(cumsum[-1])
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    q, qs = aclnn.grouped_matmul_swiglu_quant(t(x), _weight_views(wt, dev, "kmajor"), t(cumsum), t(scale), t(pt))
    torch.cuda.synchronize()
    q_ref, qs_ref = oracle.grouped_matmul_swiglu_quant(x, wt, scale, pt, cumsum, w_trans=True)
    diff = np.abs(q.cpu().numpy().astype(np.int32) - q_ref.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
    np.testing.assert_allclose(qs.cpu().numpy(), qs_ref, rtol=1e-5)


@pytest.mark.parametrize("cap_mb,K,N", [(1, 1024, 2048), (2, 1152, 2048), (1, 200, 768)])
def test_swiglu_workspace_cap_runs_in_row_bands(aclnn, oracle, dev, monkeypatch, cap_mb, K, N):
    """A cap on the fp32 SwiGLU workspace makes the operator run schedule, GEMM and requantisation once per band of rows
    (band edges fall inside groups, at empty groups and past the list's last row).  Results are those of the single band,
    bit for bit -- every row's accumulators, scale and maximum are its own -- and the workspace shrinks to the cap."""
    rng = np.random.default_rng(1234 + K)
    sizes = np.array([700, 3, 0, 0, 290, 31, 64, 65, 1, 257, 130, 0, 512, 90] + [int(v) for v in rng.integers(0, 40, 12)])
    E = len(sizes)
    cumsum = np.cumsum(sizes).astype(np.int64)
    M = int(cumsum[-1]) + 37   # rows past the last group stay untouched
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    wt = rng.integers(-127, 128, (E, N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (E, N)).astype(np.float32)
    pt = rng.uniform(0.01, 0.1, M).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    args = (t(x), _weight_views(wt, dev, "kmajor"), t(cumsum), t(scale), t(pt))

    def run():
        q = torch.full((M, N // 2), 77, dtype=torch.int8, device=dev)
        qs = torch.full((M,), -1.0, dtype=torch.float32, device=dev)
        ws = aclnn.Workspace()
        aclnn.grouped_matmul_swiglu_quant(*args, out=(q, qs), workspace=ws)
        torch.cuda.synchronize()
        return q.cpu().numpy(), qs.cpu().numpy(), ws.requested["aclnnGroupedMatmulSwigluQuant"]

    q1, qs1, ws_one = run()
    monkeypatch.setenv("OPAPI_SWIGLU_WORKSPACE_MB", str(cap_mb))
    q2, qs2, ws_banded = run()
    assert M * (N // 2) * 4 > 3 * (cap_mb << 20)          # at least three bands
    assert ws_banded < ws_one and ws_banded <= (cap_mb << 20) + 256 * (N // 2) * 4 + M * 4 * (N // 128) + (1 << 16)
    assert np.array_equal(q1, q2) and np.array_equal(qs1, qs2)
    assert (q2[int(cumsum[-1]):] == 77).all() and (qs2[int(cumsum[-1]):] == -1.0).all()
    q_ref, qs_ref = oracle.grouped_matmul_swiglu_quant(x[:int(cumsum[-1])], wt, scale, pt[:int(cumsum[-1])], cumsum, w_trans=True)
    diff = np.abs(q2[:int(cumsum[-1])].astype(np.int32) - q_ref.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
    np.testing.assert_allclose(qs2[:int(cumsum[-1])], qs_ref, rtol=1e-5)
