"""The rules that choose a kernel's shape are plain arithmetic on the host: their decisions at the sizes
they were measured at."""
from gpullama3_java_amd.csrc import lib


def test_few_tiles_are_cut_along_k_down_to_slices_of_512_columns():
    assert lib.mfma_slices(300, 2048, 8192) == 8          # 48 tiles of 128
    assert lib.mfma_slices(300, 2048, 2048) == 4          # (a slice is at least 512 columns)
    assert lib.mfma_slices(2048, 2048, 8192) == 2         # 256 tiles
    assert lib.mfma_plan(300, 2048, 8192) == (1, 8) and lib.mfma_plan(2048, 2048, 8192) == (1, 2)


def test_many_tiles_take_the_plan_with_the_fewest_idle_places():
    # 8,192 rows of the 8B layers: 512 tiles of 256 are two full rounds; nothing to gain from slices
    assert lib.mfma_plan(8192, 4096, 14336) == (2, 1) and lib.mfma_plan(8192, 4096, 4096) == (2, 1)
    # 128 tiles of 256 leave half the chip idle: two slices (measured 308 -> 265 us and 187 -> 170 us)
    assert lib.mfma_plan(2048, 4096, 14336) == (2, 2) and lib.mfma_plan(4096, 2048, 8192) == (2, 2)
    # 276 tiles of 256 are 1.08 rounds: slices fill the second (5,886 rows of the 3B layers: 474 -> 417 us)
    assert lib.mfma_plan(5886, 3072, 8192) in ((2, 2), (2, 3))
    shape, slices = lib.mfma_plan(1536, 3072, 8192)
    assert slices > 1                                     # (161 us whole, 119 to 132 us in two or three slices)
    for M in range(300, 9000, 431):
        for N, K in ((2048, 8192), (3072, 3072), (4096, 14336), (1000, 520), (3072, 272), (6144, 8)):
            shape, slices = lib.mfma_plan(M, N, K)
            assert shape in (1, 2, 5) and 1 <= slices <= 8 and (slices == 1 or K // slices >= 512)
            assert shape != 5 or slices == 1
    # tiles of 128 rows x 256 where they are one round and the others need two rounds or slices (the output projection
    # of 2,048 rows of the 3B and 8B layers: 81 -> 68 and 110 -> 97 us with the norm; 4,096 rows of the 1B layers 64 -> 60)
    assert lib.mfma_plan(2048, 3072, 3072) == (5, 1) and lib.mfma_plan(2048, 4096, 4096) == (5, 1)
    assert lib.mfma_plan(4096, 2048, 2048) == (5, 1) and lib.mfma_plan(5886, 4096, 4096) == (5, 1)
    # ... and not where the large tiles are one round themselves or K is long
    assert lib.mfma_plan(8192, 2048, 2048) == (2, 1) and lib.mfma_plan(4096, 4096, 4096) == (2, 1)
    assert lib.mfma_plan(2048, 4096, 14336) == (2, 2) and lib.mfma_plan(3072, 3072, 3072)[0] == 2


def test_decode_attention_splits_the_keys_until_every_cu_has_a_block():
    s = lib.decode_splits
    assert s(1, 32, 8, 1024) == 1 and s(8, 32, 8, 1024, 128) == 1 and s(64, 32, 8, 16384) == 1   # short; blocks enough
    assert s(8, 32, 8, 1024, 128) == 1 and s(8, 32, 8, 2048, 64) == 1                   # 128 K elements, 64 blocks
    assert s(8, 32, 8, 2048, 128) == 4 and s(8, 32, 8, 4096, 64) == 4                   # 256 K elements
    assert s(1, 32, 8, 4096) == 8 and s(1, 32, 8, 8192) == 16 and s(1, 32, 8, 32768) == 32   # few blocks: a split per 32 K elements
    assert s(1, 32, 8, 2048, 128) == 8 and s(2, 32, 8, 4096, 128) == 16
    assert s(4, 32, 8, 4096, 64) == 4 and s(4, 32, 8, 16384, 64) == 8                    # more than 16 blocks: per 64 K
    assert s(8, 32, 8, 32768) == 4 and s(16, 32, 8, 32768) == 2 and s(32, 32, 8, 32768) == 1   # 256 blocks, not more
    assert s(2, 64, 2, 100000) == 32                                  # never more than 32


def test_which_weights_a_copy_can_stand_for():
    """``lib.can_hold_once`` / ``ops.can_hold_once``: a copy in the matrix cores' order can stand for the matrix when it
    has exactly the matrix's elements over whole steps of 64 k; a weight with packed strips of 8 only must also be
    one whose products of 9 to 64 rows the kernel of whole lines takes with K in slices; any fast path switched off
    keeps both orders."""
    import torch
    from gpullama3_java_amd.parts import ops

    def weight(N, K, strips16, strips8):
        w = torch.zeros(N, K, dtype=torch.bfloat16)
        if strips16:
            w.tiled = torch.zeros(N * -(-K // 32) * 32, dtype=torch.bfloat16)
            w.tiled.tiled_for = None
        if strips8:
            w.tiled8 = torch.zeros(N * -(-K // 64) * 64, dtype=torch.bfloat16)
        return w

    assert lib.can_hold_once(weight(2048, 2048, True, False)) and lib.can_hold_once(weight(2048, 8192, False, True))
    assert not lib.can_hold_once(weight(2048, 2048, False, False))                     # no copy
    assert not lib.can_hold_once(weight(96, 96, True, False))                          # K is no whole number of steps of 64
    assert not lib.can_hold_once(weight(136, 512, True, False))                        # rows in no whole strips of 16
    assert lib.can_hold_once(weight(136, 512, False, True))                            # ... but in strips of 8
    assert ops.can_hold_once(weight(2048, 8192, False, True))                          # down projection of the 1B layers
    assert not ops.can_hold_once(weight(136, 512, False, True))                        # no slices of K for 9 to 64 rows
    assert not ops.can_hold_once(weight(136, 512, True, True))                         # (136 rows are no whole strips of 16)
    assert ops.can_hold_once(weight(128, 512, True, True))
    assert not ops.can_hold_once(weight(2048, 2048, True, False), frozenset({"once"}))
    assert not ops.can_hold_once(weight(2048, 2048, True, False), frozenset({"wide"}))
    assert not lib.held_once(weight(64, 64, True, True))


def test_which_stacked_gate_and_up_rows_stand_alone_in_operand_order():
    """``ops.gated_alone``: the up strips must follow the gate strips (N a multiple of 16), K comes in whole steps
    of 64, byte offsets of 32 bits reach all of it, and no fast path is switched off."""
    import torch
    from gpullama3_java_amd.parts import ops

    class OnGpu:                       # what the rule looks at, without a GPU
        is_cuda, dtype = True, torch.bfloat16

        def __init__(self, rows, K):
            self.shape = (rows, K)

        def dim(self):
            return 2

        def is_contiguous(self):
            return True

        def numel(self):
            return self.shape[0] * self.shape[1]

    assert ops.gated_alone(OnGpu(2 * 8192, 2048)) and ops.gated_alone(OnGpu(2 * 14336, 4096))     # 1B, 8B layers
    assert ops.gated_alone(OnGpu(2 * 48, 64))
    assert not ops.gated_alone(OnGpu(2 * 40, 64))            # 40 gate rows: the up rows would begin inside a strip
    assert not ops.gated_alone(OnGpu(2 * 48, 96))            # K in no whole steps of 64
    assert not ops.gated_alone(OnGpu(2 * 8192, 2048), frozenset({"once"}))
    assert not ops.gated_alone(OnGpu(2 * 65536, 16384))      # beyond 32-bit byte offsets
    cpu = torch.zeros(96, 64, dtype=torch.bfloat16)
    assert not ops.gated_alone(cpu)


def test_strips_slices_and_pieces_of_the_products_of_few_rows():
    """The rules that decide a decode step's kernels, at the sizes they were measured at."""
    from gpullama3_java_amd.parts import ops
    rows = lib.skinny_strip_rows
    # strips of 8 weight rows where strips of 16 would leave more than a third of the CUs without a block
    assert rows(8, 2048, 2048, lib.EPI_ADD) == 8 and rows(8, 2048, 8192, lib.EPI_ADD) == 8            # 1B output, down
    assert rows(8, 3072, 3072, lib.EPI_ADD) == 16 and rows(8, 4096, 14336, lib.EPI_ADD) == 16         # 3B, 8B: strips enough
    assert rows(12, 2048, 2048, lib.EPI_ADD) == 16 and rows(12, 2048, 8192, lib.EPI_ADD) == 8          # 9 to 16 rows: only a long K
    assert rows(40, 2048, 8192, lib.EPI_ADD) == 16 and rows(8, 2048, 2048, lib.EPI_GATED) == 16
    # the kernel of whole lines cuts K so that the chip has blocks enough, never below 512 columns a slice
    assert lib.wide_slices(2048, 2048) == 4 and lib.wide_slices(2048, 8192) == 4 and lib.wide_slices(4096, 14336) == 2
    assert lib.wide_slices(3072, 3072) == 2 and lib.wide_slices(136, 512) == 1 and lib.wide_slices(128256, 2048) == 1
    # which kernel keeps the rows of a step in registers
    assert lib.skinny_keeps_operands(8, 4096) and not lib.skinny_keeps_operands(8, 8192)
    assert lib.skinny_keeps_operands(40, 2048) and not lib.skinny_keeps_operands(40, 3072)
    # a replayed step of 66 to 128 rows is worked on in two pieces; other steps are not
    class Ctx:
        replayed = True
    assert ops.row_chunks(64, Ctx) is None and ops.row_chunks(65, Ctx) is None and ops.row_chunks(129, Ctx) is None
    assert ops.row_chunks(66, Ctx) == [(0, 33), (33, 66)] and ops.row_chunks(128, Ctx) == [(0, 64), (64, 128)]
    Ctx.replayed = False
    assert ops.row_chunks(100, Ctx) is None
    assert ops.FUSE_ROWS == 16 and ops.CHUNK_ROWS == 128
    # the gated product of few rows runs on the kernel of whole lines where it has blocks enough (and then needs no copy)
    import torch
    assert ops.gated_on_whole_lines(torch.empty(2 * 8192, 8, dtype=torch.bfloat16))
    assert not ops.gated_on_whole_lines(torch.empty(2 * 320, 8, dtype=torch.bfloat16))
    assert not ops.gated_on_whole_lines(torch.empty(2 * 8192, 8, dtype=torch.bfloat16), frozenset({"widefold"}))
