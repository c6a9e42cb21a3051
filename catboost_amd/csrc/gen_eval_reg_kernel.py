"""Writes the gfx950 assembly of the register-resident evaluate kernels.

The kernels evaluate oblivious trees of depth <= 8 (LEAVES = 64 or 256; LEAVES = 1024: depth <= 10, one
dimension, plain and six-bit forms, level tables of 32 dwords of which the first 20 are used, the two extra
levels' bits in a second index byte per document). The plain variants take models whose bins and
split indexes all fit 7 bits (no xor masks), the case of float-feature models with at most 127
used borders per feature; the "_s" variants take such models when no feature uses more than 63
borders, which lets two levels share their merge; the "_m" (mixed) variants take any bins and xor masks (one-hot splits)
and choose the compare per tree. One launch produces PITCH consecutive dimensions of the result
(1 for a one-dimensional model).

Layout of the work:
  * a wave owns one block of 256 documents and keeps the block's bins in vector registers for the
    whole launch: register B0 + b holds the dword of bucket b (byte j of lane l = document
    block * 256 + j * 64 + l), so a level of a tree costs no memory access at all. The bucket of a
    level is wave-uniform, which lets the level's compare read "register B0 + bucket" through the
    VGPR index mode (S_SET_GPR_IDX_*), the one thing the HIP compiler cannot be made to emit for a
    200-register array;
  * the waves of a workgroup share the leaf values: trees go through LDS in blocks of TREE_BLOCK
    trees (LEAVES rows of PITCH doubles per tree), double buffered; the copy of the next block is
    spread over the current block's trees and goes from global memory straight into LDS
    (global_load_lds);
  * a tree's levels come from a table of 16 dwords per tree, (bucket, (128 - splitIdx) * 0x01010101)
    per level, read with one scalar load two trees ahead; kernels for LEAVES = 64 use the first six.
    Six-bit variants: the even levels' constant is (64 - splitIdx) * 0x01010101, which puts the level's
    bit in bit 6 of every byte (all bins are below 64), next to the following level's in bit 7.
    Mixed variants: 32 dwords per tree. Bit 31 of the first dword clear: the 7-bit form above (the
    tree has no xor mask and all bins of its buckets fit 7 bits). Set: 4 dwords per level, bucket,
    xorMask, splitIdx & 0x7f (both times 0x01010101) and 0x80808080 if splitIdx < 128 else 0; the
    unsigned byte compare (bin ^ xorMask) >= splitIdx is then bit 7 of
    majority(x, (x | 0x80) - (splitIdx & 0x7f), splitIdx < 128) taken per byte, x = bin ^ xorMask;
  * the leaf gathers of a tree (four documents per lane) are issued behind its levels and consumed
    after the levels of the next tree, so their LDS latency is covered. One-dimensional kernels with
    eight registers to spare keep two sets of leaf values: a tree's gathers go out in one batch right
    behind the wait for the previous tree's (which sit in the other set and are added behind the batch),
    so that a gather has a whole tree's instructions to arrive; every sum is accumulated in
    fp64 in tree order, exactly like the CPU evaluator (cpu/evaluator_impl.cpp:362-460), and
    finished as ApplyScaleAndBias does (scale_and_bias.cpp:4-50).

Kernel arguments (80 bytes):
   0 bins        const uint32*   [docBlock][bucketCount][64]
   8 rows        const uint32*   [(treeBlocks + 2) * TREE_BLOCK][16 or 32]  (null trees behind the model's)
  16 leaves      const double*   [(treeBlocks + 2) * TREE_BLOCK][LEAVES][PITCH]
  24 out         double*         [docCount][dim]
  32 docCount    uint32          36 blockCount uint32 (ceil(docCount / 256), >= 1)
  40 treeBlocks  uint32 (>= 1)   44 flags uint32 (bit 0: add the bias)
  48 scale       double          56 bias const double* (first dimension of this launch)
  64 bucketCount uint32 (1 .. BUCKETS)                68 dim uint32
  72 first dimension of this launch uint32            76 dimensions to store uint32 (1 .. PITCH)
  80 tree blocks per slice uint32 (kernels that are not fused)
  88 map of the bins registers const uint32* (kernels that are not fused, read when flags bit 3 is set;
     96 bytes in all)
grid = (ceil(blockCount / WAVES), slices) workgroups of WAVES * 64 threads, LDS = 2 * TREE_BLOCK * LEAVES *
PITCH * 8 bytes. Slice y of the grid takes the tree blocks from y * (tree blocks per slice) on, at most that
many, and writes to out + y * docCount * dim: a small batch is spread over the chip by giving every slice
of the trees its own workgroups, which store raw sums (flags bit 2) that a second kernel adds up in slice
order. One slice (grid.y = 1, tree blocks per slice = treeBlocks) is the plain launch.

Fused variants ("cbamd_fused_..."; one-dimensional float-only models, plain and six-bit forms) take the
documents' fp32 rows instead of bins and binarize them into the bins registers themselves, so the bins
never exist in memory. Their leaf table is preceded by FUSED_CHUNKS 32 KB images of border tables, which
go through the same two LDS buffers as the tree blocks that follow them:
  * a lane owns the documents block * 256 + lane + 64 * j as before and reads its own rows, 16 bytes (four
    columns) per load, 64 bytes (a "unit" of sixteen columns = sixteen bins registers) per document and
    turn; the two units that share a 128-byte stretch of the rows are taken one right after the other;
  * a value's bin is found as the HIP binarize kernel finds it: the value's cell in the bucket's uniform
    grid of 256 cells, min(255, u32((v - lo) * scale)), indexes a byte table of search starts, and a
    branch-free binary search over the next 2^steps - 1 borders finishes the count of borders below the
    value; four columns of a document go through it side by side. steps (at most FUSED_MAX_STEPS) is
    common to the four columns of a load;
  * per unit a record of 40 dwords: sixteen lo, sixteen scale, a flags dword (bit q: the unit's q-th four
    columns need four steps, bit 4 + q: three or more, bit 8 + q: two or more, bit 16 + i: NaN counts
    as +inf in column i); behind the BUCKETS / 16 + 1 records, the units' byte offsets in a row.
Additional kernel arguments (104 bytes in all):
  80 floats const float*  88 units const uint32* [BUCKETS / 16 + 1][40] + [16]  96 row stride in bytes uint32
 100 unitCount uint32 (1 .. BUCKETS / 16)
and argument 0 is unused, argument 16 points at the border table images.

Usage: gen_eval_reg_kernel.py OUT.s
"""
import sys


LDS_BUFFER_LIMIT = 32 * 1024

# (bins registers, waves per workgroup, PITCH, LEAVES), each in a plain, a six-bit and a mixed form;
# hip_evaluator.hip lists the same variants
SHAPES = [
    (224, 4, 1, 256), (208, 4, 1, 256), (200, 4, 1, 256), (96, 8, 1, 256),
    (96, 8, 1, 64),
    (192, 4, 2, 64), (160, 4, 4, 64), (128, 4, 6, 64),
    (192, 4, 2, 256), (160, 4, 4, 256), (128, 4, 6, 256),
]
# trees of depth 9 and 10 (1024 leaf rows, one dimension): plain and six-bit forms only
DEEP_SHAPES = [(208, 4, 1, 1024), (96, 8, 1, 1024)]
VARIANTS = [shape + (mixed, six) for mixed, six in ((False, False), (False, True), (True, False)) for shape in SHAPES]
VARIANTS += [shape + (False, six) for six in (False, True) for shape in DEEP_SHAPES]
# shapes of the fused kernels (one dimension, 256 leaf rows), each in a plain and a six-bit form. The wide shape,
# and two of 64 and 80 bins registers that still run four waves per SIMD (112 and 128 registers); a model of more
# units, up to 96 buckets, runs its separate evaluate kernel at four waves per SIMD, which a fused kernel of 96
# bins registers (144: three) does not match: measured, two launches are the faster there.
FUSED_SHAPES = [(208, 4), (64, 8), (80, 8)]
# Every shape also in a form that walks six levels ("_d6": models of depth <= 6; the leaf tables keep the 256 rows
# per tree that the border images' buffers are sized for, the index reaches the first 64 of them).
FUSED_SIX_LEVEL_BUCKETS = 208
FUSED_MAX_STEPS = 4
FUSED_EXTRA_SETS = 1
FUSED_UNIT_DWORDS = 40


def fused_layout(six):
    """(buckets per border table image, bytes of a bucket's borders): the borders of the image's buckets,
    then from byte 16384 on their 256-byte tables of search starts."""
    return (64, 256) if six else (32, 512)


def fused_chunks(buckets, six):
    """Border table images in front of the leaf table: enough for `buckets`, an even number."""
    per_chunk = fused_layout(six)[0]
    chunks = (buckets + per_chunk - 1) // per_chunk
    return chunks + chunks % 2


def kernel_name(buckets, waves, pitch, leaves, mixed, six=False, fused=False, levels=None):
    if fused:
        return "cbamd_fused_b%d_w%d%s%s" % (buckets, waves, "_d6" if levels == 6 else "", "_s" if six else "")
    return "cbamd_eval_reg_b%d_w%d_p%d_l%d%s" % (buckets, waves, pitch, leaves, "_m" if mixed else "_s" if six else "")


def tree_block(pitch, leaves):
    """Trees per LDS buffer: a power of two, at most 16, buffer at most LDS_BUFFER_LIMIT bytes."""
    block = 16
    while block > 1 and block * leaves * pitch * 8 > LDS_BUFFER_LIMIT:
        block //= 2
    return block


def gen_kernel(buckets, waves, pitch, leaves, mixed, six=False, fused=False, levels=None):
    assert not (mixed and six)
    assert not fused or (pitch == 1 and leaves == 256 and not mixed and buckets % 16 == 0)
    assert levels is None or (fused and levels == 6)
    name = kernel_name(buckets, waves, pitch, leaves, mixed, six, fused, levels)
    depth = levels or {64: 6, 256: 8, 1024: 10}[leaves]
    deep = depth > 8                      # levels 8 and 9 go into a second index word
    assert not deep or (pitch == 1 and not mixed and not fused)
    row_dwords = 32 if mixed or deep else 16      # level table of a tree
    tree_row_bytes = row_dwords * 4
    rows_a, rows_b = 32, 32 + row_dwords  # the two sets of scalar registers holding level tables
    assert pitch == 1 or pitch % 2 == 0
    threads = waves * 64
    row_bytes = threads * 16              # one 16-byte piece per thread of a leaf table copy
    tree_bytes = leaves * pitch * 8
    block = tree_block(pitch, leaves)
    buf_bytes = block * tree_bytes
    lds_bytes = 2 * buf_bytes
    assert buf_bytes % row_bytes == 0 and lds_bytes <= 65536
    # A wave copies its own contiguous share of a tree block, 1 KB (16 bytes per lane) per instruction;
    # up to four instructions of a group differ only in the immediate offset, which moves the source
    # and the LDS destination alike.
    wave_bytes = buf_bytes // waves
    pieces = wave_bytes // 1024
    assert wave_bytes % 1024 == 0 and pieces >= 1
    groups = [(first, min(4, pieces - first)) for first in range(0, pieces, 4)]
    assert len(groups) <= block

    def group_step(g):
        """Distance of group g's first piece from the previous group's, the previous block's last one for g = 0."""
        if g == 0:
            return buf_bytes - groups[-1][0] * 1024
        return (groups[g][0] - groups[g - 1][0]) * 1024
    # vector registers: v0 thread, v1 lane * 4, v2 thread * 16, v3 leaf indexes, v4/v5 scratch
    lv0 = 6                               # leaf values in flight: 4 documents x pitch doubles
    ac0 = lv0 + 8 * pitch                 # the sums
    ga0 = ac0 + 8 * pitch                 # gather addresses of the four documents
    te0 = ga0 + 4                         # two scratch registers of the epilogue
    wd0 = te0 + 2                         # deep kernels: the ten-bit leaf indexes of documents 0, 1 and 2, 3 as words
    b0 = wd0 + (2 if deep else 0)         # the bins
    vgprs = b0 + buckets
    if fused:
        # registers of the binarize phase: those below the bins except v0 and v2, and 20 above the bins
        high = vgprs
        vgprs += 20
        row_off = [1, 3, 4, 5]            # byte offset of the lane's four rows from the block's first row
        srch_p = [6, 7, 8, 9]             # four searches side by side: position, border / scratch
        srch_b = [10, 11, 12, 13]
        # two sets of four 16-byte loads (first registers of the quads)
        values = [[16, 20, 24, high], [high + 4, high + 8, high + 12, high + 16]]
        assert b0 == 28
    # second set of leaf values in flight (one-dimensional kernels that have the registers for it): above the
    # bins; the fused kernels take eight of the registers that only their binarize phase uses
    def waves_per_simd(registers):
        return 512 // ((registers + 7) // 8 * 8)
    # (not where the eight registers would cost a wave per SIMD: the 96-register shape runs four)
    two_sets = pitch == 1 and block % 2 == 0 and (fused or (vgprs + 8 <= 256 and waves_per_simd(vgprs + 8) == waves_per_simd(vgprs)))
    if two_sets:
        if fused:
            lw0 = high + 8
        else:
            lw0 = vgprs
            vgprs += 8
    assert vgprs <= 256

    def lv(j, k, other=False):
        return (lw0 if other else lv0) + 2 * (j * pitch + k)

    def ac(j, k):
        return ac0 + 2 * (j * pitch + k)

    o = []
    e = o.append

    def stage(buffer_offset, g):
        """Group g of the wave's pieces of a tree block, global memory -> LDS without passing through
        registers: lane l writes 16 bytes at buffer_offset + wave * wave_bytes + piece * 1024 + l * 16 (M0
        holds the wave's base). M0 doubles as the VGPR index register, so its index-mode value is put
        back after."""
        first, count = groups[g]
        e("  s_add_u32 m0, s100, %d" % (buffer_offset + first * 1024))
        # the thread's offset moves on to the group's first piece; the instruction also fills the wait
        # state that the M0 write needs before the copy
        e("  v_add_u32_e32 v2, 0x%x, v2" % group_step(g))
        for piece in range(count):
            e("  global_load_lds_dwordx4 v2, s[26:27]%s" % (" offset:%d" % (piece * 1024) if piece else ""))

    def add_leaf_values(other=False):
        # sum + leaf as 1.0 * leaf + sum: the same single rounding, and with a constant in src0 the
        # instruction does not depend on the register index that the levels leave in M0
        for j in range(4):
            for k in range(pitch):
                e("  v_fma_f64 v[%d:%d], 1.0, v[%d:%d], v[%d:%d]" % (ac(j, k), ac(j, k) + 1, lv(j, k, other), lv(j, k, other) + 1,
                                                                      ac(j, k), ac(j, k) + 1))

    def load_rows(regs, tree):
        """Level table of tree `tree` (counted from the table position in s[6:7]) -> registers."""
        for part in range(row_dwords // 16):
            e("  s_load_dwordx16 s[%d:%d], s[6:7], 0x%x" % (regs + 16 * part, regs + 16 * part + 15,
                                                            tree * tree_row_bytes + 64 * part))

    # With eight levels the first level's sum needs no masking: each later level shifts the index
    # right by one and replaces bit 7 of every byte, so the seven low bits of the first sum leave
    # their byte one by one through bit 0, land on bit 7 of the byte below and are overwritten there.
    # Six-level kernels keep the mask: two of those bits would stay below the index.
    first_level_masked = depth < 8

    def levels_high(rows):
        """Levels 8 and 9 of a deep tree (constants (128 - splitIdx) in every form): their bits become bits 0 and
        1 of a second byte per document, and the two bytes of a document one 16-bit word: v[wd0] holds the
        indexes of documents 0 and 1, v[wd0 + 1] those of 2 and 3. The index register is set to 0 behind the
        last level, so that the instructions that follow may name vector registers in src0."""
        e("  s_set_gpr_idx_idx s%d" % (rows + 16))
        e("  v_add_u32_e64 v4, v%d, s%d" % (b0, rows + 17))
        e("  s_set_gpr_idx_idx s%d" % (rows + 18))
        e("  v_add_u32_e64 v5, v%d, s%d" % (b0, rows + 19))
        e("  s_set_gpr_idx_idx 0")
        e("  v_lshrrev_b32_e32 v4, 7, v4")
        e("  v_lshrrev_b32_e32 v5, 6, v5")
        e("  v_and_b32_e32 v4, 0x01010101, v4")
        e("  v_and_b32_e32 v5, 0x02020202, v5")
        e("  v_or_b32_e32 v4, v4, v5")
        e("  v_perm_b32 v%d, v4, v3, s24" % wd0)        # bytes: index 0 low, high, index 1 low, high
        e("  v_perm_b32 v%d, v4, v3, s25" % (wd0 + 1))

    def levels_seven_bit(rows):
        for d in range(min(depth, 8)):
            e("  s_set_gpr_idx_idx s%d" % (rows + 2 * d))
            if d == 0 and not first_level_masked:
                e("  v_add_u32_e64 v3, v%d, s%d" % (b0, rows + 2 * d + 1))
                continue
            e("  v_add_u32_e64 v4, v%d, s%d" % (b0, rows + 2 * d + 1))
            if d == 0:
                e("  v_and_b32_e32 v3, s22, v4")
            else:
                e("  v_lshrrev_b32_e32 v3, 1, v3")
                e("  v_bfi_b32 v3, s22, v4, v3")

    def levels_six_bit(rows):
        """Bins below 64 everywhere: the host gives the even levels the constant (64 - splitIdx), whose sum
        has the level's bit in bit 6 (and bit 7 clear), the odd levels (128 - splitIdx) as in the 7-bit
        form. A pair of levels is then merged into the index with one shift: five instructions for two
        levels instead of six. What the first pair leaves below its two bits goes the way the 7-bit
        form's first sum goes; six-level kernels mask it."""
        for pair in range(min(depth, 8) // 2):
            even, odd = rows + 4 * pair, rows + 4 * pair + 2
            e("  s_set_gpr_idx_idx s%d" % even)
            e("  v_add_u32_e64 v4, v%d, s%d" % (b0, even + 1))
            e("  s_set_gpr_idx_idx s%d" % odd)
            e("  v_add_u32_e64 v%d, v%d, s%d" % (3 if pair == 0 else 5, b0, odd + 1))
            if pair == 0:
                e("  v_bfi_b32 v3, s22, v3, v4")           # bit 7 of the odd level's sum over the even level's
                if first_level_masked:
                    e("  v_and_b32_e32 v3, s29, v3")
            else:
                e("  v_bfi_b32 v4, s22, v5, v4")
                e("  v_lshrrev_b32_e32 v3, 2, v3")
                e("  v_bfi_b32 v3, s29, v4, v3")

    def levels_eight_bit(rows):
        for d in range(depth):
            level = rows + 4 * d
            e("  s_set_gpr_idx_idx s%d" % level)                      # index = bits 0..7 of the bucket dword
            e("  v_xor_b32_e64 v4, v%d, s%d" % (b0, level + 1))       # x = bin ^ xorMask
            e("  v_or_b32_e32 v5, s22, v4")
            e("  v_subrev_u32_e32 v5, s%d, v5" % (level + 2))         # (x | 0x80) - (splitIdx & 0x7f), per byte
            if d == 0 and not first_level_masked:
                e("  v_bitop3_b32 v3, s%d, v4, v5 bitop3:0xe8" % (level + 3))  # majority
                continue
            e("  v_bitop3_b32 v4, s%d, v4, v5 bitop3:0xe8" % (level + 3))  # majority
            if d == 0:
                e("  v_and_b32_e32 v3, s22, v4")
            else:
                e("  v_lshrrev_b32_e32 v3, 1, v3")
                e("  v_bfi_b32 v3, s22, v4, v3")

    def fused_binarize():
        """The binarize phase of a fused kernel: fills the bins registers from the documents' rows. On
        entry the first border table image is on its way into buffer 0 and s24 holds the wave's document
        block; on exit the first tree block sits in buffer 0 and every wave has passed the barrier behind it."""
        per_chunk, border_bytes = fused_layout(six)
        units_per_chunk = per_chunk // 16
        max_units = buckets // 16
        chunks = fused_chunks(buckets, six)
        # scalar registers of the two unit records in flight: sixteen lo, sixteen scale, (flags, offset)
        rec_lo, rec_scale, rec_fo = [32, 68], [48, 84], [64, 66]
        e("  s_lshl_b32 s30, s24, 8")                 # first row of the block
        e("  s_sub_u32 s31, s12, s30")
        e("  s_add_u32 s31, s31, -1")
        e("  s_min_u32 s31, s31, 0xff")               # last row of the batch, counted from the block's first, at most 255
        e("  s_mul_hi_u32 s3, s30, s88")
        e("  s_mul_i32 s25, s30, s88")
        e("  s_add_u32 s4, s84, s25")                 # s[4:5]: the block's first row
        e("  s_addc_u32 s5, s85, s3")
        e("  v_and_b32_e32 v%d, 63, v0" % srch_p[0])
        for j in range(4):
            # rows past the last document are read as the last document
            e("  v_add_u32_e32 v%d, %d, v%d" % (row_off[j], 64 * j, srch_p[0]))
            e("  v_min_u32_e32 v%d, s31, v%d" % (row_off[j], row_off[j]))
            e("  v_mul_lo_u32 v%d, v%d, s88" % (row_off[j], row_off[j]))
        e("  s_mov_b32 s24, s86")                     # s[24:25]: unit records, s28: units of the model
        e("  s_mov_b32 s25, s87")
        e("  s_mov_b32 s28, s89")
        # the units' byte offsets in a row (they follow the records) stay in s6 .. s19 for the whole phase;
        # the arguments that sat there are loaded again behind it
        assert max_units <= 14
        offsets_at = (max_units + 1) * FUSED_UNIT_DWORDS * 4
        e("  s_load_dwordx2 s[6:7], s[24:25], 0x%x" % offsets_at)
        e("  s_load_dwordx8 s[8:15], s[24:25], 0x%x" % (offsets_at + 8))
        e("  s_load_dwordx4 s[16:19], s[24:25], 0x%x" % (offsets_at + 40))

        def load_record(n):
            unit, x = seq[n][0], n % 2
            at = unit * FUSED_UNIT_DWORDS * 4
            e("  s_load_dwordx16 s[%d:%d], s[24:25], 0x%x" % (rec_lo[x], rec_lo[x] + 15, at))
            e("  s_load_dwordx16 s[%d:%d], s[24:25], 0x%x" % (rec_scale[x], rec_scale[x] + 15, at + 64))
            e("  s_load_dwordx2 s[%d:%d], s[24:25], 0x%x" % (rec_fo[x], rec_fo[x] + 1, at + 128))

        # every unit for each of the lane's four documents: image by image, inside an image document by
        # document, so that neighbouring units of a row, which share 128-byte lines, follow each other
        seq = [(unit, j) for c in range(chunks) for j in range(4)
               for unit in range(c * units_per_chunk, min((c + 1) * units_per_chunk, max_units))]
        pending = []                      # vector memory operations in flight, oldest first

        def issue_loads(n, pieces=range(4)):
            unit, j = seq[n]
            if 0 in pieces:
                e("  s_add_u32 s30, s4, s%d" % (6 + unit))
                e("  s_addc_u32 s31, s5, 0")
            for q in pieces:
                first = value_set[n][q]
                e("  global_load_dwordx4 v[%d:%d], v%d, s[30:31]%s" % (first, first + 3, row_off[j],
                                                                      " offset:%d" % (16 * q) if q else ""))
                pending.append(("unit", n))

        def wait_loads(n):
            last = max((i for i, op in enumerate(pending) if op == ("unit", n)), default=None)
            if last is not None:
                e("  s_waitcnt vmcnt(%d)" % (len(pending) - 1 - last))
                del pending[:last + 1]

        def search_step(step, vals):
            """Step `step` (counted from the last one, 1) of the four searches: looks at the border 2^(step-1)
            places on and moves on behind it when it lies below the value."""
            size = 4 << (step - 1)
            for d in range(4):
                e("  ds_read_b32 v%d, v%d offset:%d" % (srch_b[d], srch_p[d], search_step.border_at[d] + size - 4))
            e("  s_waitcnt lgkmcnt(0)")
            for d in range(4):
                e("  v_cmp_lt_f32_e32 vcc, v%d, v%d" % (srch_b[d], vals + d))
                e("  v_cndmask_b32_e64 v%d, 0, %d, vcc" % (srch_b[d], size))
                e("  v_add_u32_e32 v%d, v%d, v%d" % (srch_p[d], srch_p[d], srch_b[d]))

        def process(n, buf):
            unit, j = seq[n]
            lo, scale, flags = rec_lo[n % 2], rec_scale[n % 2], rec_fo[n % 2]
            label = "%s_u%d_%d" % (name, unit, j)
            e("  s_waitcnt lgkmcnt(0)")                # the unit's record
            # NaN counts as +inf in the columns whose flag says so
            e("  s_lshr_b32 s3, s%d, 16" % flags)
            e("  s_cmp_eq_u32 s3, 0")
            e("  s_cbranch_scc1 %s_n" % label)
            e("  v_mov_b32_e32 v%d, 0x7f800000" % srch_b[0])
            for i in range(16):
                reg = value_set[n][i // 4] + i % 4
                e("  s_bitcmp1_b32 s%d, %d" % (flags, 16 + i))
                e("  s_cbranch_scc0 %s_n%d" % (label, i))
                e("  v_cmp_u_f32_e32 vcc, v%d, v%d" % (reg, reg))
                e("  v_cndmask_b32_e32 v%d, v%d, v%d, vcc" % (reg, reg, srch_b[0]))
                e("%s_n%d:" % (label, i))
            e("%s_n:" % label)
            for q in range(4):
                vals = value_set[n][q]
                local = (unit % units_per_chunk) * 16 + 4 * q
                search_step.border_at = [buf * buf_bytes + (local + d) * border_bytes for d in range(4)]
                for d in range(4):
                    i = 4 * q + d
                    # the value's cell in the column's grid and the search start stored for it
                    e("  v_subrev_f32_e32 v%d, s%d, v%d" % (srch_b[d], lo + i, vals + d))
                    e("  v_mul_f32_e32 v%d, s%d, v%d" % (srch_b[d], scale + i, srch_b[d]))
                    e("  v_cvt_u32_f32_e32 v%d, v%d" % (srch_b[d], srch_b[d]))
                    e("  v_min_u32_e32 v%d, 0xff, v%d" % (srch_b[d], srch_b[d]))
                    e("  ds_read_u8 v%d, v%d offset:%d" % (srch_p[d], srch_b[d],
                                                           buf * buf_bytes + 16384 + (local + d) * 256))
                e("  s_waitcnt lgkmcnt(0)")
                if not six:
                    for d in range(4):
                        e("  v_lshlrev_b32_e32 v%d, 2, v%d" % (srch_p[d], srch_p[d]))
                # the search: steps above two are rare and sit out of line
                e("  s_bitcmp1_b32 s%d, %d" % (flags, 4 + q))
                e("  s_cbranch_scc1 %s_q%d_hi" % (label, q))
                e("%s_q%d_back:" % (label, q))
                e("  s_bitcmp1_b32 s%d, %d" % (flags, 8 + q))
                e("  s_cbranch_scc0 %s_q%d_one" % (label, q))
                search_step(2, vals)
                e("%s_q%d_one:" % (label, q))
                search_step(1, vals)
                for d in range(4):
                    reg = b0 + unit * 16 + 4 * q + d
                    if j == 0:
                        e("  v_lshrrev_b32_e32 v%d, 2, v%d" % (reg, srch_p[d]))
                    else:
                        e("  v_lshl_add_u32 v%d, v%d, %d, v%d" % (reg, srch_p[d], 8 * j - 2, reg))
                out_of_line.append((label, q, vals, list(search_step.border_at), flags))

        def emit_out_of_line():
            for label, q, vals, border_at, flags in out_of_line:
                search_step.border_at = border_at
                e("%s_q%d_hi:" % (label, q))
                e("  s_bitcmp1_b32 s%d, %d" % (flags, q))
                e("  s_cbranch_scc0 %s_q%d_three" % (label, q))
                search_step(4, vals)
                e("%s_q%d_three:" % (label, q))
                search_step(3, vals)
                e("  s_branch %s_q%d_back" % (label, q))
            del out_of_line[:]

        # Two neighbouring units of a document (128 bytes of its row) are loaded together, eight loads one
        # behind the other, so that a line of the row is asked for once (the cache merges requests that
        # meet there; asked for piece by piece a line came from memory up to twice). Registers of the loads
        # in flight: the 32 below and above the bins and, while the bins registers of the last units are
        # not yet written, FUSED_EXTRA_SETS more sets of 32 among those. Inside an image the sets go round,
        # so that a pair's loads are issued that many pairs ahead of its turn; images that have no such
        # set left load, wait and search in turn (the other waves of the CU fill the wait).
        chunk_positions = [[n for n in range(len(seq)) if seq[n][0] // units_per_chunk == c] for c in range(chunks)]
        value_set = {}
        plan = []                                      # per image: (pairs of positions, sets in use, pair loaded ahead across the boundary)
        for c, positions in enumerate(chunk_positions):
            pairs = []
            for n in positions:
                if pairs and len(pairs[-1]) < 2 and seq[pairs[-1][0]][1] == seq[n][1]:
                    pairs[-1].append(n)
                else:
                    pairs.append([n])
            later_units = [u for u in range(max_units - 1, -1, -1) if u // units_per_chunk > c]
            sets = [values[0] + values[1]]
            for k in range(min(FUSED_EXTRA_SETS, len(later_units) // 2)):
                sets.append([b0 + 16 * u + 4 * q for u in later_units[2 * k:2 * k + 2] for q in range(4)])
            for k, pair in enumerate(pairs):
                for h, n in enumerate(pair):
                    value_set[n] = sets[k % len(sets)][4 * h:4 * h + 4]
            cross = bool(pairs) and len(sets) > 1 and (len(pairs) - 1) % len(sets) != 0
            plan.append((pairs, len(sets), cross))

        out_of_line = []
        load_record(0)
        if len(seq) > 1:
            load_record(1)
        e("  s_waitcnt lgkmcnt(0)")
        issued = set()
        for n in plan[0][0][0]:
            issue_loads(n)
            issued.add(n)
        e("  s_waitcnt vmcnt(0)")                      # the first image (and the first loads)
        e("  s_barrier")
        del pending[:]
        done = set(issued)                            # unit loads known to have arrived
        for c, (pairs, set_count, cross) in enumerate(plan):
            buf = c % 2
            for g in range(len(groups)):
                stage((1 - buf) * buf_bytes, g)
                pending.extend([("stage", c)] * groups[g][1])
            if pairs:
                # the model has no unit in this image: nothing to do but to pass it on
                e("  s_cmp_le_u32 s28, %d" % seq[pairs[0][0]][0])
                e("  s_cbranch_scc1 %s_c%d_end" % (name, c))
            for k, pair in enumerate(pairs):
                ahead = [p for p in pairs[k:k + set_count] if p[0] not in issued]
                if k == len(pairs) - 1 and cross and c + 1 < len(plan) and plan[c + 1][0]:
                    ahead.append(plan[c + 1][0][0])
                for p in ahead:
                    for n in p:
                        issue_loads(n)
                        issued.add(n)
                if pair[-1] in done:
                    done.difference_update(pair)
                else:
                    wait_loads(pair[-1])
                for n in pair:
                    unit, j = seq[n]
                    if unit > 0:
                        e("  s_cmp_le_u32 s28, %d" % unit)
                        e("  s_cbranch_scc1 %s_u%d_%d_skip" % (name, unit, j))
                    process(n, buf)
                    e("%s_u%d_%d_skip:" % (name, unit, j))
                    if n + 2 < len(seq):
                        load_record(n + 2)
            e("  s_branch %s_c%d_end" % (name, c))
            emit_out_of_line()
            e("%s_c%d_end:" % (name, c))
            e("  s_waitcnt vmcnt(0) lgkmcnt(0)")
            e("  s_barrier")
            if any(op[0] == "unit" for op in pending):
                done.update(op[1] for op in pending if op[0] == "unit")
            del pending[:]
        n = len(issued)
        assert n == len(seq)
        # the record and offset registers held these arguments
        e("  s_load_dwordx4 s[96:99], s[0:1], 0x40")
        e("  s_load_dwordx8 s[4:11], s[0:1], 0x0")
        e("  s_load_dwordx8 s[12:19], s[0:1], 0x20")
        e("  s_waitcnt lgkmcnt(0)")                    # the level tables are loaded through s[6:7] next

    e(".text")
    e(".globl %s" % name)
    e(".p2align 8")
    e(".type %s,@function" % name)
    e("%s:" % name)
    # s[0:1] kernarg segment, s2 workgroup id, v0 thread id
    e("  s_load_dwordx8 s[4:11], s[0:1], 0x0")
    e("  s_load_dwordx8 s[12:19], s[0:1], 0x20")
    e("  s_load_dwordx4 s[96:99], s[0:1], 0x40")
    if not fused:
        e("  s_load_dword s101, s[0:1], 0x50")         # tree blocks per slice
    if fused:
        e("  s_load_dwordx4 s[84:87], s[0:1], 0x50")   # floats, unit records
        e("  s_load_dwordx2 s[88:89], s[0:1], 0x60")   # row stride in bytes, units
    e("  v_and_b32_e32 v0, 0x3ff, v0")           # work-item ids come packed; keep x
    e("  v_lshrrev_b32_e32 v5, 6, v0")
    e("  v_and_b32_e32 v1, 63, v0")
    e("  v_lshlrev_b32_e32 v1, 2, v1")           # lane * 4: offset inside a bucket's 256 bytes
    e("  v_lshlrev_b32_e32 v2, 2, v1")           # lane * 16: offset of the lane's part of a copied piece;
    #                                              the wave's share and the first step are added below
    # gfx940 family: a lane read needs one wait state behind the VALU write of its source register;
    # the three instructions above and the s_nop keep it well clear
    e("  s_nop 1")
    e("  v_readfirstlane_b32 s20, v5")           # wave of the workgroup
    e("  s_mov_b32 s22, 0x80808080")
    if six:
        e("  s_mov_b32 s29, 0xc0c0c0c0")
    # byte j of the leaf indexes times s23 = offset of the document's leaf row in a tree's table
    # (a six-level index sits in bits 2..7 of its byte)
    # (tables of several dimensions hold a tree's values as pieces of two dimensions, each piece an array of
    # 16 bytes per leaf: a wave's 16-byte gathers then spread over all sixteen groups of four LDS banks, which
    # leaf rows of 32 bytes would not)
    e("  s_mov_b32 s23, %d" % ((8 if pitch == 1 else 16) >> max(8 - depth, 0)))
    e("  s_mul_i32 s100, s20, %d" % wave_bytes)  # offset of the wave's share of a tree block
    # one step back: every group of copies steps forward first
    e("  s_sub_u32 s28, s100, %d" % group_step(0))
    e("  v_add_u32_e32 v2, s28, v2")
    e("  s_waitcnt lgkmcnt(0)")
    if not fused:
        # the slice of the trees that this row of the grid takes (s3: workgroup id y)
        e("  s_mul_i32 s24, s3, s101")               # its first tree block
        e("  s_sub_u32 s25, s14, s24")
        e("  s_min_u32 s14, s25, s101")              # its tree blocks
        e("  s_mul_i32 s25, s24, %d" % (block * tree_row_bytes))
        e("  s_add_u32 s6, s6, s25")
        e("  s_addc_u32 s7, s7, 0")
        e("  s_mul_hi_u32 s28, s24, %d" % buf_bytes)
        e("  s_mul_i32 s25, s24, %d" % buf_bytes)
        e("  s_add_u32 s8, s8, s25")
        e("  s_addc_u32 s9, s9, s28")
        e("  s_mul_i32 s25, s12, s97")               # values of one slice: docCount * dim (below 2^29)
        e("  s_lshl_b32 s25, s25, 3")
        e("  s_mul_hi_u32 s28, s25, s3")
        e("  s_mul_i32 s25, s25, s3")
        e("  s_add_u32 s10, s10, s25")
        e("  s_addc_u32 s11, s11, s28")
    # first tree block -> buffer 0
    e("  s_mov_b32 s26, s8")
    e("  s_mov_b32 s27, s9")
    for g in range(len(groups)):
        stage(0, g)
    # document block of this wave; waves past the last block redo the last one and store nothing
    e("  s_mul_i32 s21, s2, %d" % waves)
    e("  s_add_u32 s21, s21, s20")
    e("  s_add_u32 s24, s13, -1")
    e("  s_min_u32 s24, s21, s24")
    if fused:
        fused_binarize()
    else:
        # (the level table registers are free until the first tables are loaded)
        e("  s_lshl_b32 s25, s96, 8")                # bytes of bins per document block
        e("  s_mul_hi_u32 s31, s24, s25")
        e("  s_mul_i32 s30, s24, s25")
        e("  s_add_u32 s32, s4, s30")
        e("  s_addc_u32 s33, s5, s31")
        e("  s_add_u32 s28, s96, -1")
        e("  s_bitcmp1_b32 s15, 3")
        e("  s_cbranch_scc1 %s_mapped" % name)
        for i in range(buckets):
            # registers past the model's bucket count reload the last bucket and are never indexed
            e("  s_min_u32 s24, %d, s28" % i)
            e("  s_lshl_b32 s24, s24, 8")
            e("  s_add_u32 s34, s32, s24")
            e("  s_addc_u32 s35, s33, 0")
            e("  global_load_dword v%d, v1, s[34:35]" % (b0 + i))
        if True:
            # Flags bit 3: the bins registers follow a map, one dword per register: bits 0..15 the bucket it
            # is loaded from, bits 16.. what becomes of the bins there: 0 as they are, 1 min(bin, 127), 2
            # max(bin - 127, 0). A float bucket with more than 127 values then takes two registers, and a level
            # "bin >= s" reads the first (s <= 127) or the second (with s - 127): every tree without xor
            # masks runs in the 7-bit form. The map has ceil(BUCKETS / 16) * 16 entries.
            e("  s_branch %s_loaded" % name)
            e("%s_mapped:" % name)
            e("  s_load_dwordx2 s[52:53], s[0:1], 0x58")
            e("  s_mov_b32 s25, 0x7f7f7f7f")
            batches = (buckets + 15) // 16
            for batch in range(batches):
                e("  s_waitcnt lgkmcnt(0)")
                e("  s_load_dwordx16 s[36:51], s[52:53], 0x%x" % (64 * batch))
                e("  s_waitcnt lgkmcnt(0)")
                for k in range(16):
                    i = 16 * batch + k
                    if i >= buckets:
                        break
                    e("  s_and_b32 s24, s%d, 0xffff" % (36 + k))
                    e("  s_lshl_b32 s24, s24, 8")
                    e("  s_add_u32 s34, s32, s24")
                    e("  s_addc_u32 s35, s33, 0")
                    e("  global_load_dword v%d, v1, s[34:35]" % (b0 + i))
            e("  s_waitcnt vmcnt(0)")
            for batch in range(batches):
                e("  s_load_dwordx16 s[36:51], s[52:53], 0x%x" % (64 * batch))
                e("  s_waitcnt lgkmcnt(0)")
                for k in range(16):
                    i = 16 * batch + k
                    if i >= buckets:
                        break
                    reg = b0 + i
                    label = "%s_map%d" % (name, i)
                    e("  s_lshr_b32 s24, s%d, 16" % (36 + k))
                    e("  s_cmp_eq_u32 s24, 0")
                    e("  s_cbranch_scc1 %s" % label)
                    # bytes of 128 and more -> 0xff
                    e("  v_and_b32_e32 v4, 0x80808080, v%d" % reg)
                    e("  v_lshrrev_b32_e32 v5, 7, v4")
                    e("  v_sub_u32_e32 v5, v4, v5")
                    e("  v_or_b32_e32 v4, v4, v5")
                    e("  s_cmp_eq_u32 s24, 1")
                    e("  s_cbranch_scc1 %s_low" % label)
                    e("  v_and_b32_e32 v5, 0x7f7f7f7f, v%d" % reg)      # those bytes: (bin & 127) + 1 = bin - 127
                    e("  v_add_u32_e32 v5, 0x1010101, v5")
                    e("  v_and_b32_e32 v%d, v4, v5" % reg)
                    e("  s_branch %s" % label)
                    e("%s_low:" % label)
                    e("  v_bfi_b32 v%d, v4, s25, v%d" % (reg, reg))      # those bytes: 127
                    e("%s:" % label)
            e("%s_loaded:" % name)
    load_rows(rows_a, 0)
    load_rows(rows_b, 1)
    for r in list(range(lv0, ga0)) + (list(range(lw0, lw0 + 8)) if two_sets else []):
        e("  v_mov_b32_e32 v%d, 0" % r)          # leaf values in flight and the sums
    # a launch that continues the sums of earlier trees takes them from `out`
    e("  s_bitcmp1_b32 s15, 1")
    e("  s_cbranch_scc0 %s_fresh" % name)
    e("  v_and_b32_e32 v5, 63, v0")
    e("  s_lshl_b32 s24, s21, 8")
    e("  v_add_u32_e32 v5, s24, v5")
    for j in range(4):
        e("  v_add_u32_e32 v%d, %d, v5" % (te0, 64 * j))
        e("  v_cmp_gt_u32_e32 vcc, s12, v%d" % te0)
        e("  s_and_saveexec_b64 s[30:31], vcc")
        e("  v_mul_lo_u32 v%d, v%d, s97" % (te0 + 1, te0))
        e("  v_add_lshl_u32 v%d, v%d, s98, 3" % (te0 + 1, te0 + 1))
        for k in range(pitch):
            if k > 0:
                e("  s_cmp_gt_u32 s99, %d" % k)
                e("  s_cbranch_scc0 %s_taken_%d" % (name, j))
            e("  global_load_dwordx2 v[%d:%d], v%d, s[10:11] offset:%d" % (ac(j, k), ac(j, k) + 1, te0 + 1, 8 * k))
        e("%s_taken_%d:" % (name, j))
        e("  s_mov_b64 exec, s[30:31]")
    e("%s_fresh:" % name)
    e("  s_waitcnt vmcnt(0) lgkmcnt(0)")
    e("  s_barrier")
    e("  s_set_gpr_idx_on s22, 0x1")             # src0 of VALU instructions becomes index relative
    # every wave warms its own share of a tree block's level tables, every WARM_WAYS-th 64-byte line
    # from line (wave mod WARM_WAYS) on: s[30:31] = table + that line
    warm_lines = block * tree_row_bytes // 64
    warm_ways = min(waves, warm_lines)
    assert warm_ways & (warm_ways - 1) == 0 and warm_lines % warm_ways == 0
    e("  s_and_b32 s28, s20, %d" % (warm_ways - 1))
    e("  s_lshl_b32 s28, s28, 6")
    e("  s_add_u32 s30, s6, s28")
    e("  s_addc_u32 s31, s7, 0")
    if deep:
        # byte selectors of the two index words (s24 and s25 are free from here to the epilogue)
        e("  s_mov_b32 s24, 0x05010400")
        e("  s_mov_b32 s25, 0x07030602")
    e("%s_loop:" % name)
    for buf in range(2):
        for i in range(block):
            rows = rows_a if i % 2 == 0 else rows_b
            if mixed:
                label = "%s_t%d_%d" % (name, buf, i)
                e("  s_bitcmp1_b32 s%d, 31" % rows)
                e("  s_cbranch_scc1 %s_x" % label)
                levels_seven_bit(rows)
                e("  s_branch %s_j" % label)
                e("%s_x:" % label)
                levels_eight_bit(rows)
                e("%s_j:" % label)
            elif six:
                levels_six_bit(rows)
            else:
                levels_seven_bit(rows)
            if deep:
                levels_high(rows)
            tree_offset = buf * buf_bytes + i * tree_bytes

            def gather_address(j):
                if deep:
                    e("  v_mul_u32_u24_sdwa v%d, s23, v%d dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_%d"
                      % (ga0 + j, wd0 + j // 2, j % 2))
                else:
                    e("  v_mul_u32_u24_sdwa v%d, s23, v3 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_%d"
                      % (ga0 + j, j))
            if two_sets:
                # The trees of a block alternate between the two sets of leaf values (a block has an even number
                # of trees, so the first tree of a block finds the last one's values in the second set). The wait
                # sits right in front of the tree's own gathers: the previous tree's had its levels and addresses to
                # arrive, and so had the next tree's row. Gathers in one batch, sums behind them: interleaved they
                # took longer (1.137 against 1.090 ms per 4M documents and 1000 trees).
                mine = i % 2 == 1
                for j in range(4):
                    gather_address(j)
                e("  s_waitcnt lgkmcnt(0)")
                for j in range(4):
                    e("  ds_read_b64 v[%d:%d], v%d offset:%d" % (lv(j, 0, mine), lv(j, 0, mine) + 1, ga0 + j, tree_offset))
                load_rows(rows, buf * block + i + 2)
                add_leaf_values(not mine)
            else:
                # previous tree's leaf values have arrived (and so has the next tree's row)
                e("  s_waitcnt lgkmcnt(0)")
                add_leaf_values()
                for j in range(4):
                    gather_address(j)
                    if pitch == 1:
                        e("  ds_read_b64 v[%d:%d], v%d offset:%d" % (lv(j, 0), lv(j, 0) + 1, ga0 + j, tree_offset))
                    else:
                        for k in range(0, pitch, 2):
                            e("  ds_read_b128 v[%d:%d], v%d offset:%d" % (lv(j, k), lv(j, k) + 3, ga0 + j,
                                                                         tree_offset + (k // 2) * leaves * 16))
                load_rows(rows, buf * block + i + 2)
            # copy of the next tree block into the other buffer, spread over this block's trees
            staged = False
            for g in range(len(groups)):
                if g * block // len(groups) == i:
                    stage((1 - buf) * buf_bytes, g)
                    staged = True
            if staged:
                e("  s_mov_b32 m0, 0x1000")      # index mode value again: src0 relative, index 0
            if i == 0:
                # the rows of the next tree block are pulled into the scalar cache now, so that the
                # per-tree row loads of that block do not each wait for a miss. The waves of a workgroup
                # share the cache and reach this point together, so each touches a share of the lines
                # (a scalar load is dear here: sixteen per wave and block cost 5 % of the launch)
                for k in range(warm_lines // warm_ways):
                    e("  s_load_dword s3, s[30:31], 0x%x" % ((buf * block + block + 2) * tree_row_bytes
                                                            + 64 * warm_ways * k))
        # every wave is done reading this buffer and writing the other one
        e("  s_waitcnt vmcnt(0) lgkmcnt(0)")
        e("  s_barrier")
        e("  s_add_u32 s14, s14, -1")
        e("  s_cmp_eq_u32 s14, 0")
        e("  s_cbranch_scc1 %s_done" % name)
    e("  s_add_u32 s6, s6, %d" % (2 * block * tree_row_bytes))
    e("  s_addc_u32 s7, s7, 0")
    e("  s_add_u32 s30, s30, %d" % (2 * block * tree_row_bytes))
    e("  s_addc_u32 s31, s31, 0")
    e("  s_branch %s_loop" % name)
    e("%s_done:" % name)
    add_leaf_values(two_sets)                # the last tree of a block: second set
    e("  s_set_gpr_idx_off")
    e("  s_bitcmp1_b32 s15, 2")                  # raw sums for a launch that continues them
    e("  s_cbranch_scc1 %s_store" % name)
    # scale, bias of the launch's dimensions (rows registers are free now)
    for k in range(pitch):
        e("  s_load_dwordx2 s[%d:%d], s[18:19], 0x%x" % (32 + 2 * k, 33 + 2 * k, 8 * k))
    for j in range(4):
        for k in range(pitch):
            e("  v_mul_f64 v[%d:%d], s[16:17], v[%d:%d]" % (ac(j, k), ac(j, k) + 1, ac(j, k), ac(j, k) + 1))
    e("  s_waitcnt lgkmcnt(0)")
    e("  s_bitcmp1_b32 s15, 0")
    e("  s_cbranch_scc0 %s_store" % name)
    for j in range(4):
        for k in range(pitch):
            e("  v_add_f64 v[%d:%d], v[%d:%d], s[%d:%d]" % (ac(j, k), ac(j, k) + 1, ac(j, k), ac(j, k) + 1,
                                                             32 + 2 * k, 33 + 2 * k))
    e("%s_store:" % name)
    e("  v_and_b32_e32 v5, 63, v0")
    e("  s_lshl_b32 s24, s21, 8")
    e("  v_add_u32_e32 v5, s24, v5")
    for j in range(4):
        e("  v_add_u32_e32 v%d, %d, v5" % (te0, 64 * j))
        e("  v_cmp_gt_u32_e32 vcc, s12, v%d" % te0)
        e("  s_and_saveexec_b64 s[30:31], vcc")
        e("  v_mul_lo_u32 v%d, v%d, s97" % (te0 + 1, te0))               # document * dim
        e("  v_add_lshl_u32 v%d, v%d, s98, 3" % (te0 + 1, te0 + 1))     # + first dimension, in bytes
        for k in range(pitch):
            if k > 0:
                e("  s_cmp_gt_u32 s99, %d" % k)
                e("  s_cbranch_scc0 %s_stored_%d" % (name, j))
            e("  global_store_dwordx2 v%d, v[%d:%d], s[10:11] offset:%d" % (te0 + 1, ac(j, k), ac(j, k) + 1, 8 * k))
        e("%s_stored_%d:" % (name, j))
        e("  s_mov_b64 exec, s[30:31]")
    e("  s_endpgm")
    e(".Lend_%s:" % name)
    e(".size %s, .Lend_%s-%s" % (name, name, name))
    e("")
    e(".rodata")
    e(".p2align 6")
    e(".amdhsa_kernel %s" % name)
    e("  .amdhsa_group_segment_fixed_size %d" % lds_bytes)
    e("  .amdhsa_private_segment_fixed_size 0")
    e("  .amdhsa_kernarg_size %d" % (104 if fused else 96))
    e("  .amdhsa_user_sgpr_count 2")
    e("  .amdhsa_user_sgpr_kernarg_segment_ptr 1")
    e("  .amdhsa_system_sgpr_workgroup_id_x 1")
    e("  .amdhsa_system_sgpr_workgroup_id_y 1")
    e("  .amdhsa_system_sgpr_workgroup_id_z 0")
    e("  .amdhsa_system_vgpr_workitem_id 0")
    e("  .amdhsa_next_free_vgpr %d" % vgprs)
    e("  .amdhsa_next_free_sgpr 102")
    e("  .amdhsa_accum_offset %d" % ((vgprs + 3) // 4 * 4))
    e("  .amdhsa_reserve_vcc 1")
    e("  .amdhsa_float_round_mode_32 0")
    e("  .amdhsa_float_round_mode_16_64 0")
    e("  .amdhsa_float_denorm_mode_32 3")
    e("  .amdhsa_float_denorm_mode_16_64 3")
    e("  .amdhsa_dx10_clamp 1")
    e("  .amdhsa_ieee_mode 1")
    e(".end_amdhsa_kernel")
    e("")
    meta = """  - .agpr_count: 0
    .args:
      - {.address_space: global, .offset: 0, .size: 8, .value_kind: global_buffer}
      - {.address_space: global, .offset: 8, .size: 8, .value_kind: global_buffer}
      - {.address_space: global, .offset: 16, .size: 8, .value_kind: global_buffer}
      - {.address_space: global, .offset: 24, .size: 8, .value_kind: global_buffer}
      - {.offset: 32, .size: 4, .value_kind: by_value}
      - {.offset: 36, .size: 4, .value_kind: by_value}
      - {.offset: 40, .size: 4, .value_kind: by_value}
      - {.offset: 44, .size: 4, .value_kind: by_value}
      - {.offset: 48, .size: 8, .value_kind: by_value}
      - {.address_space: global, .offset: 56, .size: 8, .value_kind: global_buffer}
      - {.offset: 64, .size: 4, .value_kind: by_value}
      - {.offset: 68, .size: 4, .value_kind: by_value}
      - {.offset: 72, .size: 4, .value_kind: by_value}
      - {.offset: 76, .size: 4, .value_kind: by_value}
%s    .group_segment_fixed_size: %d
    .kernarg_segment_align: 8
    .kernarg_segment_size: %d
    .max_flat_workgroup_size: %d
    .name: %s
    .private_segment_fixed_size: 0
    .sgpr_count: 108
    .sgpr_spill_count: 0
    .symbol: %s.kd
    .uniform_work_group_size: 1
    .uses_dynamic_stack: false
    .vgpr_count: %d
    .vgpr_spill_count: 0
    .wavefront_size: 64
""" % ("""      - {.address_space: global, .offset: 80, .size: 8, .value_kind: global_buffer}
      - {.address_space: global, .offset: 88, .size: 8, .value_kind: global_buffer}
      - {.offset: 96, .size: 4, .value_kind: by_value}
      - {.offset: 100, .size: 4, .value_kind: by_value}
""" if fused else """      - {.offset: 80, .size: 4, .value_kind: by_value}
      - {.offset: 84, .size: 4, .value_kind: by_value}
      - {.address_space: global, .offset: 88, .size: 8, .value_kind: global_buffer}
""", lds_bytes, 104 if fused else 96, threads, name, name, vgprs)
    return "\n".join(o), meta


def generate():
    parts = ['.amdgcn_target "amdgcn-amd-amdhsa--gfx950"', ".amdhsa_code_object_version 6", ""]
    metas = []
    for buckets, waves, pitch, leaves, mixed, six in VARIANTS:
        text, meta = gen_kernel(buckets, waves, pitch, leaves, mixed, six)
        parts.append(text)
        metas.append(meta)
    for buckets, waves in FUSED_SHAPES:
        for six in (False, True):
            for levels in (None, 6) if buckets <= FUSED_SIX_LEVEL_BUCKETS else (None,):
                text, meta = gen_kernel(buckets, waves, 1, 256, False, six, fused=True, levels=levels)
                parts.append(text)
                metas.append(meta)
    parts.append(".amdgpu_metadata")
    parts.append("---")
    parts.append("amdhsa.kernels:")
    parts.extend(m.rstrip("\n") for m in metas)
    parts.append("amdhsa.target: amdgcn-amd-amdhsa--gfx950")
    parts.append("amdhsa.version:")
    parts.append("  - 1")
    parts.append("  - 2")
    parts.append("...")
    parts.append(".end_amdgpu_metadata")
    return "\n".join(parts) + "\n"


if __name__ == "__main__":
    with open(sys.argv[1], "w") as f:
        f.write(generate())
