"""The shape rules that choose among kernels (pure functions of sizes): no GPU needed."""

import pytest


@pytest.fixture(scope="module")
def ops():
    from liyab_amd.kernels import ops as o

    return o


def test_parts_of_k_are_whole_and_none_is_empty(ops):
    """A product cut over K: every part holds whole units of 64 and at least one of them, for
    every shape the rules answer for."""
    for M in (1, 3, 8, 16, 17, 24, 32, 33, 48, 64, 65, 128, 200, 512, 2048):
        for N in (16, 100, 768, 1024, 1600, 2304, 4096, 4800, 8192, 16384, 50257):
            for K in (8, 64, 72, 192, 768, 1024, 1600, 3072, 4096, 6400, 8192, 16384):
                units = (K + 63) // 64
                for parts in (ops.k_parts(M, N, K), ops.tiled_k_parts(M, N, K)):
                    assert 1 <= parts <= 16
                    per = (units + parts - 1) // parts
                    assert (parts - 1) * per < units, (M, N, K, parts)
                if ops.k_parts(M, N, K) > 1:
                    assert M <= 32 and K % 8 == 0
                if ops.tiled_k_parts(M, N, K) > 1:
                    assert M > 16 and (M > 32 or N > 2048) and K % 64 == 0


def test_attention_split_plan(ops):
    """Decode attention in splits: powers of two up to 8, a split keeping 128 keys or more of the
    longest context, workgroups of 4 waves; one split when the context is short."""
    for n_tokens in (1, 2, 8, 9, 16, 17, 32):
        for n_head in (1, 3, 12, 25):
            for bucket in (256, 512, 1024, 2048, 8192, 32768):
                splits, waves = ops.decode_split_plan(n_tokens, n_head, bucket)
                assert splits in (1, 2, 4, 8) and waves in (4, 16)
                assert waves == 4 or (n_tokens * n_head <= 32 and bucket // splits >= 1024)
                assert splits == 1 or bucket // splits >= 128
                assert ops.att_parts_takes(n_tokens, splits, 64)
    assert ops.decode_split_plan(1, 12, 256)[0] == 2 and ops.decode_split_plan(1, 12, 1024)[0] == 8
    assert ops.decode_split_plan(16, 12, 1024)[0] == 4
    assert ops.decode_split_plan(1, 12, 32768) == (8, 16) and ops.decode_split_plan(8, 12, 32768) == (8, 4)


def test_attention_plan_of_tokens_that_finish_themselves(ops):
    """Decode attention that merges its own splits: 1, 4, 8 or 16 splits (two never pay), a split
    keeping 128 keys or more of the longest context, pairs x splits within 256 workgroups; cut
    keys go on 4 waves, uncut ones on 4, 8 or 16."""
    for n_tokens in (1, 2, 4, 8, 9, 17, 32, 64, 300):
        for n_head in (1, 3, 12, 25, 32):
            for bucket in (64, 256, 512, 1024, 2048, 4096, 8192, 131072):
                splits, waves = ops.decode_plan(n_tokens, n_head, bucket)
                assert splits in (1, 4, 8, 16) and waves in (4, 8, 16)
                if splits > 1:
                    assert waves == (8 if bucket // splits >= 1024 else 4) and bucket // splits >= 128 and n_tokens * n_head * splits <= 256
    assert ops.decode_plan(1, 32, 1024) == (8, 4) and ops.decode_plan(1, 12, 4096) == (16, 4)
    assert ops.decode_plan(8, 25, 1024) == (1, 8) and ops.decode_plan(4, 25, 4096) == (1, 16)
    assert ops.decode_plan(64, 12, 1024) == (1, 4) and ops.decode_plan(1, 12, 256) == (1, 4)


def test_tiled_parts_of_one_tile_of_rows(ops):
    """33 to 64 rows added to the stream: few output features in 4 parts from an inner size of
    3,072 on; many output features while 64 x 64 tiles x parts stay within 256 workgroups."""
    assert ops.tiled_k_parts(64, 768, 3072) == 4 and ops.tiled_k_parts(64, 768, 768) == 1
    assert ops.tiled_k_parts(64, 4096, 16384) == 4 and ops.tiled_k_parts(40, 4096, 4096) == 4
    assert ops.tiled_k_parts(64, 8192, 8192) == 2 and ops.tiled_k_parts(64, 16384, 4096) == 1
    assert ops.tiled_k_parts(32, 4096, 16384) == 2 and ops.tiled_k_parts(17, 4096, 4096) == 2 and ops.tiled_k_parts(24, 8192, 8192) == 1
    assert ops.tiled_k_parts(16, 4096, 16384) == 1 and ops.tiled_k_parts(32, 768, 3072) == 1


def test_what_the_folded_norm_takes(ops):
    assert ops.skinny_ln_takes(1, 64) and ops.skinny_ln_takes(32, 2048)
    assert not ops.skinny_ln_takes(33, 768) and not ops.skinny_ln_takes(8, 2056) and not ops.skinny_ln_takes(8, 100)
    assert ops.norm_takes_planes(768) and not ops.norm_takes_planes(777) and ops.norm_takes_planes(16384) and not ops.norm_takes_planes(16388)


def test_attention_tile_of_a_step():
    """Steps whose long portions hold few tokens take query tiles of 64, others of 128; short
    portions (taken token by token) do not count."""
    from liyab_amd.parts import attention as step

    assert step.attn_tile_for([1, 1, 1]) == step.ATTN_TILE_FEW
    assert step.attn_tile_for([256, 1, 8]) == step.ATTN_TILE_FEW
    assert step.attn_tile_for([1024]) == step.ATTN_TILE_FEW
    assert step.attn_tile_for([1024, 9]) == step.ATTN_TILE
    assert step.attn_tile_for([1024, 1024]) == step.ATTN_TILE
    assert step.attn_tile_for([1024] + [8] * 40) == step.ATTN_TILE_FEW


def test_attention_plans_its_own_words_of_a_step():
    """Attention's planner: a step of single tokens needs no words and is keyed by the context's
    bucket; a step with long portions gets its tiles (the one that ends latest first) and the
    short portions' rows, laid out natively, and a key that fixes their counts."""
    import ctypes

    import numpy as np

    from liyab_amd.parts import StepFacts
    from liyab_amd.parts.attention import Attention, AttentionStepPlanner

    planner = Attention.step_planner
    assert isinstance(planner, AttentionStepPlanner) and planner.name == "attention"

    def facts(q_lens, first):
        q = np.array(q_lens, dtype=np.intc)
        f = np.array(first, dtype=np.intc)
        return StepFacts(n_tokens=int(q.sum()), n_seqs=len(q), q_lens=q, first_pos=f, state_slots=np.arange(len(q), dtype=np.intc),
                         max_q_len=int(q.max()), max_context=int((q + f).max()), page_size=16)

    p = planner.plan(facts([1, 8, 3], [300, 10, 0]))
    assert p.key == ("decode", 512) and p.n_words == 0 and p.recurs and p.make(None).mode == "decode"
    p = planner.plan(facts([100, 2, 70, 9], [0, 40, 200, 5]))
    # tiles of 64: 100 -> 64 + 36, 70 -> 64 + 6, 9 -> 9; the short one's two rows are taken one by one
    assert p.key == ("prefill", 512, 5, 64, 2) and p.n_words == 4 * 5 + 2 and not p.recurs
    words = np.full(p.n_words, -7, dtype=np.int32)
    p.fill(words.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
    tiles = words[:20].reshape(5, 4).tolist()
    # (request, first row, first position, queries), ordered by the position a tile ends at
    assert tiles == [[2, 166, 264, 6], [2, 102, 200, 64], [0, 64, 64, 36], [0, 0, 0, 64], [3, 172, 5, 9]]
    assert words[20:].tolist() == [100, 101]
    # the same sizes cut another way give the same key when they fall into the same tiles
    assert planner.plan(facts([90, 2, 80, 9], [10, 40, 190, 5])).key == p.key


def test_what_makes_two_layers_one_kind_and_how_a_recorded_list_gets_another_layers_addresses():
    """Layers run from one recorded list of launches when their blocks are made of the same parts
    with the same constants (tensors aside) and every part says it is `replayable`; the list's words
    that lie inside the recorded layer's tensors become the same places of the other layer's."""
    import numpy as np
    import torch

    from liyab_amd.models.decoder import _OTHER, _Recorded, _describe

    class Part:
        replayable = True

        def __init__(self, scale, w):
            self.scale, self.w, self.names = scale, w, {"b": [w, None]}

    class Block:
        replayable = True

        def __init__(self, part):
            self.part, self.label = part, "x"

    class Foreign:
        def __init__(self):
            self.t = torch.zeros(2)

    a, b = torch.zeros(4, 3), torch.ones(4, 3)
    ta, tb, tc = [], [], []
    ka, kb = _describe(Block(Part(0.5, a)), ta, set()), _describe(Block(Part(0.5, b)), tb, set())
    assert ka == kb and ka is not _OTHER and [t.data_ptr() for t in ta] == [a.data_ptr()] * 2 and len(tb) == 2
    assert _describe(Block(Part(0.25, a)), tc, set()) != ka  # a constant of its own
    assert _describe(Block(Part(0.5, torch.zeros(4, 4))), [], set()) != ka  # another shape
    assert _describe(Block(Foreign()), [], set()) is _OTHER  # a part that does not say it may be replayed
    own = Block(Part(0.5, a))
    own.part.loop = own
    assert _describe(own, [], set()) is _OTHER  # an object met twice
    # a list whose words 2 and 5 point into the first and the second tensor of the recorded layer; word 7 is
    # a size that happens to lie in the first tensor's range and stays what it is
    bases = np.array([1000, 5000], dtype=np.uint64)
    words = np.array([7, 3, 1000 + 16, 999, 6000, 5000, 1000 + 64, 1008], dtype=np.uint64)
    addresses = np.array([False, False, True, True, True, True, False, False])
    rec = _Recorded(words, addresses, bases, [64, 100], None)
    assert rec.usable and rec.positions.tolist() == [2, 5] and rec.offsets.tolist() == [16, 0]
    assert rec.for_layer(np.array([20000, 90000], dtype=np.uint64)).tolist() == [7, 3, 20016, 999, 6000, 90000, 1064, 1008]
    assert not _Recorded(np.array([1], dtype=np.uint64), np.array([True]), np.array([1000, 1032], dtype=np.uint64), [64, 8], None).usable  # overlapping tensors


def test_padded_sizes_of_steps_with_prompt_portions():
    """The rows of a step in which some request brings more than one token: multiples of 16 up to 64,
    of 64 up to 1,024, of 128 beyond; never fewer than the tokens, never a whole unit more."""
    from liyab_amd.engine.step import padded_rows

    assert [padded_rows(n) for n in (2, 16, 17, 33, 48, 64, 65, 500, 1024, 1025, 2048)] == [16, 16, 32, 48, 48, 64, 128, 512, 1024, 1152, 2048]
    for n in range(1, 3000):
        unit = 16 if n <= 64 else 64 if n <= 1024 else 128
        assert n <= padded_rows(n) < n + unit and padded_rows(n) % unit == 0 and padded_rows(padded_rows(n)) == padded_rows(n)
