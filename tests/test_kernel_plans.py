"""Host-side decisions about kernel launches (CPU): key splits of the decode attention, pieces of
a sampled row, and which matrix-product kernel a tuned table sends a product to."""

import torch

from torchllms_amd.kernels import attention_ops, ops, products


def test_decode_splits_cover_the_range_and_stay_under_a_cu_s_share_of_blocks():
    for head_dim, per_cu in ((32, 3), (64, 3), (128, 2), (256, 1)):
        for n_tokens in (1, 2, 3, 8, 17, 64, 200):
            for n_kv_heads in (1, 2, 8):
                for longest in (1, 15, 256, 1000, 8192, 70000, 131072):
                    for uneven in (False, True):
                        split, n_splits = ops.plan_decode_splits(n_tokens, n_kv_heads, longest, head_dim, uneven=uneven)
                        assert split % 64 == 0 and split >= 128
                        assert n_splits >= 1 and (n_splits - 1) * split < max(longest, 1) <= n_splits * split
                        if uneven:
                            assert split <= attention_ops.DECODE_UNEVEN_SPLIT == 512
                        elif longest >= 4096 and split == 1024:
                            pass  # long contexts: no split beyond 1,024 keys, however many blocks that makes
                        elif n_splits > 1:
                            # (few long rows at head size 128 aim at one block a CU)
                            at_a_time = 256 * (1 if head_dim == 128 and n_tokens * n_kv_heads <= 32 else per_cu)
                            # never more blocks than the CUs take at a time, unless the shortest split allowed is reached
                            assert split == 128 or n_tokens * n_kv_heads * n_splits <= at_a_time
                            # and no fewer splits than that allows: one split more would be too many
                            shorter = split - 64
                            assert shorter < 128 or n_tokens * n_kv_heads * -(-longest // shorter) > at_a_time or -(-longest // shorter) == n_splits
    # head sizes with fewer bytes a key take more blocks a CU
    assert ops.plan_decode_splits(8, 8, 2176, 128) == (320, 7)
    assert ops.plan_decode_splits(8, 8, 2176, 64) == (192, 12)
    assert ops.plan_decode_splits(8, 4, 8192, 256) == (1024, 8)


def test_a_sampled_row_is_cut_only_when_rows_are_few_and_long():
    assert ops.sample_chunks(1, 128256) == 15 and ops.sample_chunks(8, 128256) == 15
    assert ops.sample_chunks(64, 128256) == 4 and ops.sample_chunks(256, 128256) == 1
    assert ops.sample_chunks(1, 8191) == 1 and ops.sample_chunks(1, 32000) == 3 and ops.sample_chunks(0, 128256) == 15


def test_the_tuned_table_decides_per_shape_rows_and_use():
    w = torch.zeros(96, 256, dtype=torch.bfloat16)
    x = torch.zeros(40, 256, dtype=torch.bfloat16)
    keys = [(96, 256, b, use) for b in (8, 64, 128) for use in ops.LINEAR_USES]
    saved = {k: products.LINEAR_CHOICE[k] for k in keys if k in products.LINEAR_CHOICE}
    try:
        for k in keys:
            products.LINEAR_CHOICE.pop(k, None)
        assert ops.linear_choice(x, w) is None  # 40 rows, never measured: the library
        assert ops.linear_choice(x[:8], w) == ("stream", 0)  # 8 rows, never measured: the size rule
        products.LINEAR_CHOICE[(96, 256, 64, "plain")] = ("wide", 1, 2, 3)
        products.LINEAR_CHOICE[(96, 256, 64, "glu")] = ("wide", 2, 1, 3)
        products.LINEAR_CHOICE[(96, 256, 8, "plain")] = None
        assert ops.linear_choice(x, w) == ("wide", 1, 2, 3) and ops.linear_choice(x, w, "glu") == ("wide", 2, 1, 3)
        assert ops.linear_choice(x, w, "qkv") is None and ops.linear_choice(x[:8], w) is None
        assert ops.linear_choice(x[:33], w) == ("wide", 1, 2, 3)  # 33 to 64 rows share a bucket
        assert ops.linear_choice(torch.zeros(65, 256, dtype=torch.bfloat16), w) is None  # the next bucket, never measured
        assert ops.linear_choice(torch.zeros(129, 256, dtype=torch.bfloat16), w) is None  # too many rows
        assert ops.linear_choice(torch.zeros(40, 192, dtype=torch.bfloat16), torch.zeros(96, 192, dtype=torch.bfloat16)) is None  # K % 128
        assert ops.linear_choice(x.float(), w.float()) is None
    finally:
        for k in keys:
            products.LINEAR_CHOICE.pop(k, None)
        products.LINEAR_CHOICE.update(saved)


def test_which_candidates_are_charged_a_kernel_of_their_own_for_the_second_half():
    stream, whole, split = ("stream", 4), ("wide", 2, 1, 3), ("wide", 1, 4, 3)
    for choice in (None, stream, whole, split):
        assert products.fuses_tail(choice, "plain")
    # the streaming product adds itself to the residual rows and leaves the norm's statistics; the library cannot
    assert [products.fuses_tail(c, "sum") for c in (None, stream, whole, split)] == [False, True, True, True]
    assert [products.fuses_tail(c, "glu") for c in (None, stream, whole, split)] == [False, True, True, False]
    assert [products.fuses_tail(c, "qkv") for c in (None, stream, whole, split)] == [False, True, False, True]


def test_which_launches_of_the_wide_kernel_fit_lds():
    assert ops.wide_fits(64, 2, 3) and ops.wide_fits(128, 1, 3) and ops.wide_fits(128, 2, 2) and not ops.wide_fits(128, 2, 3)
    assert ops.wide_fits(20, 2, 3) and ops.wide_fits(65, 1, 2)


def test_the_table_survives_a_file(tmp_path):
    saved = dict(products.LINEAR_CHOICE)
    try:
        products.LINEAR_CHOICE.clear()
        products.LINEAR_CHOICE.update({(96, 256, 64, "plain"): ("wide", 2, 1, 3), (96, 256, 8, "glu"): ("stream", 4, 8),
                                       (96, 256, 8, "plain"): None, (512, 128, 1, "qkv"): ("stream", 0)})
        table = ops.kernel_table()
        assert table == {"96,256,8,glu": ["stream", 4, 8], "96,256,8,plain": None, "96,256,64,plain": ["wide", 2, 1, 3],
                         "512,128,1,qkv": ["stream", 0]}
        assert ops.kernel_table([((96, 256), "plain")]) == {"96,256,8,plain": None, "96,256,64,plain": ["wide", 2, 1, 3]}
        ops.save_kernel_table(tmp_path / "t.json")
        before = dict(products.LINEAR_CHOICE)
        ops.clear_kernel_table()
        assert products.LINEAR_CHOICE == {}
        ops.load_kernel_table(tmp_path / "t.json")
        assert products.LINEAR_CHOICE == before
    finally:
        products.LINEAR_CHOICE.clear()
        products.LINEAR_CHOICE.update(saved)


def test_libraries_built_in_the_tree_match_their_sources():
    """A library built before its source was last edited is compiled again at its next use, on the GPU
    box, where the time counts: build again after every change (``__graft_entry__.build()``).  A
    tree without built libraries (a fresh checkout) has nothing to compare."""
    from torchllms_amd.kernels import build

    assert build.stale_libraries() == []


def test_launch_plans_take_the_device_s_own_figures(monkeypatch):
    """Compute units and LDS size come from the device (the target's published figures where there is
    no GPU, as here): a GPU with half the CUs gets half the splits, one with less LDS fewer buffers."""
    from torchllms_amd.kernels import lib

    assert lib.device_facts() == (256, 160 * 1024)
    assert ops.plan_decode_splits(1, 8, 8192) == (256, 32) and ops.plan_decode_splits(8, 8, 2176) == (320, 7)
    assert ops.wide_fits(64, 2, 3) and ops.rmsnorm_max_hidden() == 40704
    monkeypatch.setattr(lib, "_facts", (128, 64 * 1024))
    assert ops.plan_decode_splits(1, 8, 8192) == (512, 16) and ops.plan_decode_splits(8, 8, 2176) == (576, 4)  # half the blocks at a time
    assert not ops.wide_fits(64, 2, 3) and ops.wide_fits(32, 1, 2) and ops.rmsnorm_max_hidden() == 16128


def test_a_head_size_without_matrix_core_kernels_is_reported_once(caplog):
    """A bfloat16 model whose head size only the plain attention kernel takes runs, right and slowly:
    the attention part says so, once per shape, when the engine asks it about its sizes."""
    import logging

    from torchllms_amd.config.spec import PartSpec
    from torchllms_amd.parts import MIXERS

    def part(head_dim, heads=6, kv=3):
        return MIXERS.build(PartSpec("attention", dict(
            hidden_size=96, num_heads=heads, num_kv_heads=kv, head_dim=head_dim, qkv_bias=False, softmax_scale=head_dim ** -0.5, window=0,
            position=PartSpec("rope", dict(head_dim=head_dim, rotary_dim=head_dim, theta=100.0, scaling=None)))))

    with caplog.at_level(logging.WARNING, logger="torchllms_amd"):
        part(64).check_sizes(torch.bfloat16)
        part(96).check_sizes(torch.float32)
        assert not caplog.records
        part(96).check_sizes(torch.bfloat16)
        part(96).check_sizes(torch.bfloat16)
        assert len(caplog.records) == 1 and "head size 96" in caplog.text and "decode steps and prompts run the plain kernel" in caplog.text
        part(256, heads=16, kv=1).check_sizes(torch.bfloat16)  # 16 query heads per kv head: prompts only
        assert len(caplog.records) == 2 and "; decode steps run the plain kernel" in caplog.records[1].getMessage()


def test_near_ties_of_the_measurement_are_decided_by_rule_not_by_the_stopwatch():
    """Candidates within 4% of the fastest count as equal; among them one that does the whole use in its own
    kernels wins over one that needs a kernel behind it, a kernel of the package over the library, and the
    candidates' fixed order decides the rest: the table, and with it the bfloat16 bits, does not flip from
    run to run on a tie."""
    lib, split, whole = None, ("wide", 1, 2, 3), ("wide", 2, 1, 3)
    assert products.pick([(lib, 17.9), (split, 18.4), (whole, 22.0)], "qkv") == split  # rotates in its second kernel
    assert products.pick([(lib, 18.4), (split, 17.9)], "qkv") == split
    assert products.pick([(lib, 17.0), (split, 18.4)], "qkv") is lib  # 8% apart: no tie
    assert products.pick([(lib, 50.0), (whole, 50.5), (split, 50.2)], "glu") == whole  # the gate ends a whole product
    assert products.pick([(lib, 10.0), (split, 10.3), (whole, 10.2)], "sum") == split  # first of the package's in the list
    assert products.pick([(lib, 10.0)], "plain") is lib
