"""The launch plans are plain functions of shapes: what the kernels' host checks rely on holds
for every shape (no empty split, whole chunks and pages, bounds on the number of splits)."""
import itertools

from minfer_amd.kernels import ops


def test_skinny_plan_covers_k_without_empty_splits():
    for m, n, k, target in itertools.product((1, 8, 9, 16, 17, 40, 64), (96, 3584, 4608, 37888, 152064),
                                             (64, 200, 256, 3584, 8192, 18944), (64, 256, 1024)):
        splits, per = ops.skinny_plan(m, n, k, target_blocks=target)
        assert splits >= 1 and per % 256 == 0
        assert splits * per >= k, (m, n, k, splits, per)
        assert (splits - 1) * per < k, (m, n, k, splits, per)        # the last split has work
        if m <= 16 and k < 8192:
            assert splits == 1
        else:
            assert splits * ((n + 127) // 128) <= max(target, (n + 127) // 128), (m, n, k, splits)


def test_skinny_plan_choices_at_the_model_shapes():
    """At most 8 rows against a long K: one kernel where a CU's share of the weight rows fills its
    tiles (3584 and 8192 rows over 256 CUs), the staged K-split kernel where it does not (5120)."""
    assert ops.skinny_plan(8, 3584, 18944, target_blocks=256)[0] == 1
    assert ops.skinny_plan(8, 8192, 29568, target_blocks=256)[0] == 1
    assert ops.skinny_plan(1, 5120, 27648, target_blocks=256)[0] > 1
    assert ops.skinny_plan(9, 3584, 18944, target_blocks=256)[0] > 1
    assert ops.skinny_plan(16, 37888, 3584, target_blocks=256)[0] == 1
    # K of 8192 is held in registers where SwiGLU (or a norm) is folded in: one kernel up to 16 rows
    assert ops.skinny_plan(16, 59136, 8192, target_blocks=256, swiglu=True)[0] == 1
    assert ops.skinny_plan(16, 8192, 8192, target_blocks=256)[0] > 1
    assert ops.skinny_plan(12, 300, 8192, target_blocks=256, swiglu=True)[0] > 1      # too few weight rows for it


def test_tile_plan():
    """The tile product's plan for every shape is one the kernels take: a K split only for the
    variants that have one, in whole chunks of 256 with no empty part, the direct-to-LDS kernel only
    for K in 64s, no SwiGLU epilogue on the 192-wide tile."""
    for m, n, k, epi, aligned in itertools.product((65, 128, 200, 512, 1024, 2048, 5977, 8192), (96, 3584, 4608, 37888),
                                                   (64, 200, 256, 3584, 18944), (ops.EPI_F32, ops.EPI_SWIGLU),
                                                   (True, False)):
        if epi == ops.EPI_SWIGLU and n % 64:
            continue
        variant, splits, per = ops.tile_plan(m, n, k, epi, aligned and k % 8 == 0, n_cu=256)
        assert variant in (2, 9, 12, 13, 15)
        if variant in (12, 13, 15):
            assert aligned and k % 64 == 0
        assert variant != 15 or epi != ops.EPI_SWIGLU
        if splits == 1:
            assert per == k
            continue
        assert variant in (2, 12) and per % 256 == 0 and per >= 512
        assert splits * per >= k and (splits - 1) * per < k
        if variant == 12:
            assert m >= 768 and per >= 2048 and splits <= 8 and epi != ops.EPI_SWIGLU
        else:
            tiles = ((m + 127) // 128) * ((n + 127) // 128)
            assert tiles < 256 and splits * tiles <= 512


def test_split_plan_of_the_32_bit_attention():
    for n_tok, nk, group, hd, max_len in itertools.product((1, 8, 64, 300), (1, 2, 4), (1, 5, 7), (16, 128, 256),
                                                           (1, 64, 100, 4096, 32768)):
        n_splits, split_len = ops.split_plan(n_tok, nk, group, hd, max_len)
        assert 1 <= n_splits <= 64
        assert split_len % ops.PAGE == 0 and split_len > 0
        assert n_splits * split_len >= max_len
        assert (n_splits - 1) * split_len < max_len                   # the last split has keys


def test_decode_split_plan_bounds():
    for n_tok, nk, group, max_len in itertools.product((1, 8, 64, 300), (1, 2, 4), (1, 5, 7, 17), (1, 64, 4096, 32768)):
        places, n = ops.decode_split_plan(n_tok, nk, group, max_len, target_blocks=256)
        assert 1 <= n <= places <= 32
        assert n == 1 or n * 256 <= max_len + 255
        assert places == n or (1 < n_tok <= 64 and n > 1 and max_len >= 8192 and places == min(4 * n, 32))
    plan = lambda *a: ops.decode_split_plan(*a, target_blocks=256)
    assert plan(1, 4, 7, 32768) == (32, 32) and plan(64, 4, 7, 32768) == (1, 1)
    assert plan(8, 4, 7, 32768) == (32, 8)          # shares in proportion to the keys
    assert plan(8, 4, 7, 4096) == (8, 8)
    assert ops.decode_split_plan(8, 4, 7, 4096, target_blocks=64) == (2, 2)        # a chip of 64 CUs splits less


def test_plan_linear_names_the_kernels_of_the_model_shapes():
    """Which kernel a product takes, as the library decides it (nothing is launched): the decode
    shapes of the 7B, 32B and 72B widths get the kernels the design describes, and widths off the
    family's (896, 1024, 2560, 6144) a named path of their own."""
    p = lambda *a, **k: ops.plan_linear(*a, n_cu=256, **k)["kernel"]
    for h, inter, qkv in ((3584, 18944, 4608), (5120, 27648, 7168), (8192, 29568, 10240)):
        for m in (1, 8, 16):
            assert p(m, qkv, h, normed=True) == "stationary16_kernel(norm)"
            assert p(m, 2 * inter, h, swiglu=True, normed=True) == "stationary16_kernel(norm)"
            assert p(m, 152064, h, normed=True) == "stationary16_kernel(norm)"
        assert p(8, h, h, accumulate=True) == ("stationary16_kernel" if h <= 5120 else "rolling16_kernel")
        assert p(64, 2 * inter, h, swiglu=True) == "panel_kernel" and p(64, 152064, h) == "panel_kernel"
        # the ring form needs K in whole chunks of 256 (29568 is 115.5 of them)
        assert p(64, h, inter, accumulate=True) == ("skinny_ring_kernel" if inter % 256 == 0 else "skinny_kernel")
        assert p(2048, 2 * inter, h, swiglu=True) == "tile_dma_kernel<256>"
        assert p(40, qkv, h, normed=True) == ""                       # no fold above 16 rows: norm, then product
    assert p(8, 3584, 18944, accumulate=True) == "rolling16_kernel"
    # a prompt of 2,048 tokens at the 7B widths: 256-wide tiles of q|k|v (144) and o (112) would leave
    # half of the 256 CUs idle, so 192 tiles of 256 x 192 and 224 of 256 x 128; down has K to split
    assert p(2048, 4608, 3584, out_bf16=True) == "tile_dma_kernel<192>"
    assert p(2048, 3584, 3584, accumulate=True) == "tile_dma_kernel<128>"
    assert p(2048, 3584, 18944, accumulate=True) == "tile_dma_kernel<256>(split K)"
    assert p(8192, 4608, 3584, out_bf16=True) == "tile_dma_kernel<192>"       # 768 tiles: three whole rounds
    assert p(4096, 3584, 3584, accumulate=True) == "tile_dma_kernel<256>"     # 224 tiles: one round nearly full
    assert p(4096, 37888, 3584, swiglu=True) == "tile_dma_kernel<256>"
    assert p(2048, 3584, 3584 + 8, accumulate=True) == "tile_kernel<128,128>"      # K not in 64s
    assert p(200, 3584, 18944, accumulate=True) == "tile_kernel<128,128>(split K)"
    # other widths: multiples of 256 that are instantiated take the register-resident kernel, the
    # rest the rolling one; unaligned operands the guarded ones
    for k in (1024, 2560, 3072, 6144, 7168):
        assert p(4, 4096, k, normed=True) == "stationary16_kernel(norm)", k
    # a width of 896 (the narrowest model of the family) runs as seven waves of four steps
    assert p(4, 4096, 896, normed=True) == "stationary16_kernel(norm)" and p(4, 4096, 896) == "stationary16_kernel"
    assert p(4, 4096, 640, normed=True) == "" and p(4, 4096, 640) == "rolling16_kernel"
    assert p(4, 4096, 1280) == "rolling16_kernel"                       # 5 x 256: not instantiated
    assert p(4, 4096, 900, aligned=False) == "skinny16_kernel"
    assert p(4, 100, 1024) == "rolling16_kernel"                        # too few weight rows to go round
    assert p(30, 4096, 900, aligned=False) == "skinny_kernel"
    for ns in ops.STATIONARY_NS:
        assert ops.stationary_shape(4096, 256 * ns, True) and p(2, 4096, 256 * ns, normed=True) != ""
    assert not ops.stationary_shape(4096, 256 * 5) and not ops.stationary_shape(4096, 256 * 33, True)


def test_shared_query_tiles_cover_every_page_once():
    """The host's list of workgroups for the prompt attention: every block of 128 queries appears
    with all its shares or alone, a share's pages are at most the load asked for (unless the cap on
    shares binds), the longest entries come first, and without long blocks there is no list."""
    import torch
    from minfer_amd.engine.batch import StepContext

    def ctx(new, start):
        n = sum(new)
        return StepContext(cache=None, n_tokens=n, n_seqs=len(new), token_ids=torch.zeros(n, dtype=torch.int32),
                           positions=None, seq_of_tok=None, cu_seqlens=None, start_pos=None, slot_ids=None,
                           logit_rows=None, page_tables={}, max_len=0, max_new=max(new), all_decode=False,
                           host_new=list(new), host_start=list(start))

    for new, start, window, load, cap in (([1500, 260, 40], [600, 0, 0], 0, 4, 8), ([64], [30000], 0, 26, 8),
                                          ([2048], [0], 0, 15, 8), ([300, 17], [900, 5000], 700, 4, 3)):
        got = ctx(new, start).shared_query_tiles(128, 64, window, 1, 1 << 19, 2, load, cap)      # the least load binds
        assert got is not None
        seqs, q0s, words, n_slots, most = (x.tolist() if hasattr(x, "tolist") else x for x in got)
        tiles = {}
        for b, q0, w in zip(seqs, q0s, words):
            tiles.setdefault((b, q0), []).append(w)
        assert sorted(tiles) == sorted((b, q0) for b, n in enumerate(new) for q0 in range(0, n, 128))
        slots = set()
        for (b, q0), ws in tiles.items():
            last_key = start[b] + min(q0 + 128, new[b]) - 1
            first_key = max(0, start[b] + q0 - window + 1) if window else 0
            pages = last_key // 64 - first_key // 64 + 1
            if ws == [0]:
                assert pages <= load
                continue
            n = (ws[0] >> 8) & 255
            assert sorted(w & 255 for w in ws) == list(range(n)) and {(w >> 8) & 255 for w in ws} == {n}
            assert len({w >> 16 for w in ws}) == 1 and 2 <= n <= min(cap, most)
            assert n == cap or -(-pages // n) <= load
            slots.add(ws[0] >> 16)
        assert slots == set(range(n_slots))
    assert ctx([100, 30], [0, 0]).shared_query_tiles(128, 64, 0, 1, 1 << 19, 2, 4, 8) is None
    # the even share binds: 64 tokens on 30,000 are 470 pages; 28 heads over 512 workgroups at once
    # give each at most 26 of them, 4 heads give each at most 4: layers with other head counts get
    # plans of their own from the same step
    c = ctx([64], [30000])
    a = c.shared_query_tiles(128, 64, 0, 28, 256, 2, 4, 64)
    b = c.shared_query_tiles(128, 64, 0, 4, 256, 2, 4, 64)
    assert a[4] == -(-470 // 26) and b[4] == 64 and c.shared_query_tiles(128, 64, 0, 28, 256, 2, 4, 64) is a
    # no sharing where it cannot gain: a whole prompt of 2,048 tokens with 28 heads keeps every CU
    # busy for as long as its longest block takes (32 pages against an even 30 a CU); with 2 heads
    # the CUs would idle behind the longest blocks
    assert ctx([2048], [0]).shared_query_tiles(128, 64, 0, 28, 256, 2, 4, 8) is None
    assert ctx([2048], [0]).shared_query_tiles(128, 64, 0, 2, 256, 2, 4, 8) is not None
    assert ctx([128] * 8, [2000] * 8).shared_query_tiles(128, 64, 0, 28, 256, 2, 4, 8) is None
    assert ctx([512], [4096]).shared_query_tiles(128, 64, 0, 28, 256, 2, 4, 8) is not None


def test_prefill_tile_takes_a_group_of_heads_together():
    """Rows of the prompt attention are (token, head of the kv group) pairs, 128 a workgroup: as many
    whole tokens as fit beside all heads of the group; a group with more heads than rows goes in chunks."""
    assert ops.prefill_tile(28, 4, 128) == (18, 7, 4)          # the 7B shape: 126 of 128 rows in use
    assert ops.prefill_tile(6, 6, 64) == (128, 1, 6)           # one head a group: 128 tokens
    assert ops.prefill_tile(64, 8, 128) == (16, 8, 8)
    assert ops.prefill_tile(40, 8, 256) == (25, 5, 8)
    assert ops.prefill_tile(130, 1, 16) == (1, 128, 2)         # 130 heads: a token's heads in two workgroups
    for nh, nk, hd in itertools.product((1, 3, 12, 28, 64, 300), (1, 2, 4), (16, 48, 128, 256)):
        if nh % nk:
            continue
        tq, gh, per_tile = ops.prefill_tile(nh, nk, hd)
        group = nh // nk
        assert 1 <= gh <= group and tq >= 1 and tq * gh <= 128
        assert per_tile == nk * -(-group // gh)


def test_skinny_plan_keeps_a_small_matrix_in_one_kernel():
    assert ops.skinny_plan(8, 2048, 11008, target_blocks=256, tiled=True)[0] == 1      # the 3B shape's down product
    assert ops.skinny_plan(16, 2048, 11008, target_blocks=256, tiled=True)[0] > 1
    assert ops.skinny_plan(8, 5120, 13824, target_blocks=256, tiled=True)[0] > 1       # the 14B shape's: 141 MB
