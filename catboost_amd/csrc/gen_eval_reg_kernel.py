"""Writes the gfx950 assembly of the register-resident evaluate kernels.

The kernels evaluate oblivious trees of depth <= 8 of a one-dimensional model whose bins and
split indexes all fit 7 bits (no xor masks), the case of float-feature models with at most 127
used borders per feature.

Layout of the work:
  * a wave owns one block of 256 documents and keeps the block's bins in vector registers for the
    whole launch: register B0 + b holds the dword of bucket b (byte j of lane l = document
    block * 256 + j * 64 + l), so a level of a tree costs no memory access at all. The bucket of a
    level is wave-uniform, which lets the level's compare read "register B0 + bucket" through the
    VGPR index mode (S_SET_GPR_IDX_*), the one thing the HIP compiler cannot be made to emit for a
    200-register array;
  * the waves of a workgroup share the leaf values: trees go through LDS in blocks of TREE_BLOCK
    trees (256 doubles per tree), double buffered; the copy of the next block is spread over the
    current block's trees and goes from global memory straight into LDS (global_load_lds);
  * a tree's levels come from a table of 16 dwords per tree, (bucket, (128 - splitIdx) * 0x01010101)
    per level, read with one scalar load two trees ahead;
  * the four leaf gathers of a tree are issued behind its levels and consumed after the levels of
    the next tree, so their LDS latency is covered; every document's sum is accumulated in fp64 in
    tree order, exactly like the CPU evaluator (cpu/evaluator_impl.cpp:362-460), and finished as
    ApplyScaleAndBias does (scale_and_bias.cpp:4-50).

Kernel arguments (72 bytes):
   0 bins        const uint32*   [docBlock][bucketCount][64]
   8 rows        const uint32*   [(treeBlocks + 2) * TREE_BLOCK][16]    (null trees behind the model's)
  16 leaves      const double*   [(treeBlocks + 2) * TREE_BLOCK][256]
  24 out         double*         [docCount]
  32 docCount    uint32          36 blockCount uint32 (ceil(docCount / 256), >= 1)
  40 treeBlocks  uint32 (>= 1)   44 flags uint32 (bit 0: add the bias)
  48 scale       double          56 bias double
  64 bucketCount uint32 (1 .. BUCKETS)
grid = ceil(blockCount / WAVES) workgroups of WAVES * 64 threads, LDS = 2 * TREE_BLOCK * 2048 bytes.

Usage: gen_eval_reg_kernel.py OUT.s
"""
import sys

TREE_BLOCK = 16
TREE_BYTES = 2048
BUF_BYTES = TREE_BLOCK * TREE_BYTES
LDS_BYTES = 2 * BUF_BYTES
ROW_BYTES = 64
B0 = 32  # first bins register

# (bins registers, waves per workgroup)
VARIANTS = [(208, 4), (96, 8)]


def kernel_name(buckets, waves):
    return "cbamd_eval_reg_b%d_w%d" % (buckets, waves)


def gen_kernel(buckets, waves):
    name = kernel_name(buckets, waves)
    threads = waves * 64
    row_bytes = threads * 16              # one 16-byte piece per thread
    chunks = BUF_BYTES // row_bytes       # pieces of a tree block per thread
    assert 1 <= chunks <= TREE_BLOCK
    vgprs = B0 + buckets
    assert vgprs <= 256
    o = []
    e = o.append

    def stage(lds_offset):
        """One piece of the leaf table, global memory -> LDS without passing through registers:
        lane l of wave w writes 16 bytes at lds_offset + w * 1024 + l * 16 (M0 holds the wave's
        base). M0 doubles as the VGPR index register, so its index-mode value is put back after."""
        e("  s_add_u32 m0, s68, %d" % lds_offset)
        e("  s_nop 0")
        e("  global_load_lds_dwordx4 v2, s[26:27]")
        e("  s_add_u32 s26, s26, %d" % row_bytes)
        e("  s_addc_u32 s27, s27, 0")

    e(".text")
    e(".globl %s" % name)
    e(".p2align 8")
    e(".type %s,@function" % name)
    e("%s:" % name)
    # s[0:1] kernarg segment, s2 workgroup id, v0 thread id
    e("  s_load_dwordx8 s[4:11], s[0:1], 0x0")
    e("  s_load_dwordx8 s[12:19], s[0:1], 0x20")
    e("  s_load_dword s29, s[0:1], 0x40")
    e("  v_and_b32_e32 v0, 0x3ff, v0")           # work-item ids come packed; keep x
    e("  v_lshrrev_b32_e32 v5, 6, v0")
    e("  v_and_b32_e32 v1, 63, v0")
    e("  v_lshlrev_b32_e32 v1, 2, v1")           # lane * 4: offset inside a bucket's 256 bytes
    e("  v_lshlrev_b32_e32 v2, 4, v0")           # thread * 16: offset of the thread's piece of a copy
    # gfx940 family: a lane read needs one wait state behind the VALU write of its source register;
    # the three instructions above and the s_nop keep it well clear
    e("  s_nop 1")
    e("  v_readfirstlane_b32 s20, v5")           # wave of the workgroup
    e("  s_mov_b32 s22, 0x80808080")
    e("  s_mov_b32 s23, 3")
    e("  s_lshl_b32 s68, s20, 10")               # LDS offset of the wave's part of a copied piece
    e("  s_waitcnt lgkmcnt(0)")
    # first tree block -> buffer 0
    e("  s_mov_b32 s26, s8")
    e("  s_mov_b32 s27, s9")
    for c in range(chunks):
        stage(c * row_bytes)
    # document block of this wave; waves past the last block redo the last one and store nothing
    e("  s_mul_i32 s21, s2, %d" % waves)
    e("  s_add_u32 s21, s21, s20")
    e("  s_add_u32 s24, s13, -1")
    e("  s_min_u32 s24, s21, s24")
    e("  s_lshl_b32 s25, s29, 8")                # bytes of bins per document block
    e("  s_mul_hi_u32 s31, s24, s25")
    e("  s_mul_i32 s30, s24, s25")
    e("  s_add_u32 s64, s4, s30")
    e("  s_addc_u32 s65, s5, s31")
    e("  s_add_u32 s28, s29, -1")
    for i in range(buckets):
        # registers past the model's bucket count reload the last bucket and are never indexed
        e("  s_min_u32 s24, %d, s28" % i)
        e("  s_lshl_b32 s24, s24, 8")
        e("  s_add_u32 s66, s64, s24")
        e("  s_addc_u32 s67, s65, 0")
        e("  global_load_dword v%d, v1, s[66:67]" % (B0 + i))
    e("  s_load_dwordx16 s[32:47], s[6:7], 0x0")
    e("  s_load_dwordx16 s[48:63], s[6:7], 0x%x" % ROW_BYTES)
    for r in range(6, 22):
        e("  v_mov_b32_e32 v%d, 0" % r)          # leaf values in flight and the four sums
    e("  s_waitcnt vmcnt(0) lgkmcnt(0)")
    e("  s_barrier")
    e("  s_set_gpr_idx_on s23, 0x1")             # src0 of VALU instructions becomes index relative
    e("%s_loop:" % name)
    for buf in range(2):
        for i in range(TREE_BLOCK):
            rows = 32 if i % 2 == 0 else 48
            for d in range(8):
                e("  s_set_gpr_idx_idx s%d" % (rows + 2 * d))
                e("  v_add_u32_e64 v4, v%d, s%d" % (B0, rows + 2 * d + 1))
                if d == 0:
                    e("  v_and_b32_e32 v3, s22, v4")
                else:
                    e("  v_lshrrev_b32_e32 v3, 1, v3")
                    e("  v_bfi_b32 v3, s22, v4, v3")
            e("  s_set_gpr_idx_idx 0")
            # previous tree's leaf values have arrived (and so has the next tree's row)
            e("  s_waitcnt lgkmcnt(0)")
            for j in range(4):
                a = 14 + 2 * j
                l = 6 + 2 * j
                e("  v_add_f64 v[%d:%d], v[%d:%d], v[%d:%d]" % (a, a + 1, a, a + 1, l, l + 1))
            for j in range(4):
                l = 6 + 2 * j
                e("  v_lshlrev_b32_sdwa v%d, s23, v3 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_%d"
                  % (22 + j, j))
                e("  ds_read_b64 v[%d:%d], v%d offset:%d" % (l, l + 1, 22 + j, buf * BUF_BYTES + i * TREE_BYTES))
            e("  s_load_dwordx16 s[%d:%d], s[6:7], 0x%x" % (rows, rows + 15, (buf * TREE_BLOCK + i + 2) * ROW_BYTES))
            # copy of the next tree block into the other buffer, one piece per tree
            if i < chunks:
                stage((1 - buf) * BUF_BYTES + i * row_bytes)
                e("  s_mov_b32 m0, 0x1000")      # index mode value again: src0 relative, index 0
            if i == 0:
                # the rows of the next tree block are pulled into the scalar cache now, so that the
                # per-tree row loads of that block do not each wait for a miss
                for k in range(TREE_BLOCK):
                    e("  s_load_dword s3, s[6:7], 0x%x" % ((buf * TREE_BLOCK + TREE_BLOCK + 2 + k) * ROW_BYTES))
        # every wave is done reading this buffer and writing the other one
        e("  s_waitcnt vmcnt(0) lgkmcnt(0)")
        e("  s_barrier")
        e("  s_add_u32 s14, s14, -1")
        e("  s_cmp_eq_u32 s14, 0")
        e("  s_cbranch_scc1 %s_done" % name)
    e("  s_add_u32 s6, s6, %d" % (2 * TREE_BLOCK * ROW_BYTES))
    e("  s_addc_u32 s7, s7, 0")
    e("  s_branch %s_loop" % name)
    e("%s_done:" % name)
    for j in range(4):
        a = 14 + 2 * j
        l = 6 + 2 * j
        e("  v_add_f64 v[%d:%d], v[%d:%d], v[%d:%d]" % (a, a + 1, a, a + 1, l, l + 1))
    e("  s_set_gpr_idx_off")
    for j in range(4):
        a = 14 + 2 * j
        e("  v_mul_f64 v[%d:%d], s[16:17], v[%d:%d]" % (a, a + 1, a, a + 1))
    e("  s_bitcmp1_b32 s15, 0")
    e("  s_cbranch_scc0 %s_store" % name)
    for j in range(4):
        a = 14 + 2 * j
        e("  v_add_f64 v[%d:%d], v[%d:%d], s[18:19]" % (a, a + 1, a, a + 1))
    e("%s_store:" % name)
    e("  v_and_b32_e32 v5, 63, v0")
    e("  s_lshl_b32 s24, s21, 8")
    e("  v_add_u32_e32 v5, s24, v5")
    for j in range(4):
        a = 14 + 2 * j
        e("  v_add_u32_e32 v30, %d, v5" % (64 * j))
        e("  v_cmp_gt_u32_e32 vcc, s12, v30")
        e("  s_and_saveexec_b64 s[30:31], vcc")
        e("  v_lshlrev_b32_e32 v31, 3, v30")
        e("  global_store_dwordx2 v31, v[%d:%d], s[10:11]" % (a, a + 1))
        e("  s_mov_b64 exec, s[30:31]")
    e("  s_endpgm")
    e(".Lend_%s:" % name)
    e(".size %s, .Lend_%s-%s" % (name, name, name))
    e("")
    e(".rodata")
    e(".p2align 6")
    e(".amdhsa_kernel %s" % name)
    e("  .amdhsa_group_segment_fixed_size %d" % LDS_BYTES)
    e("  .amdhsa_private_segment_fixed_size 0")
    e("  .amdhsa_kernarg_size 72")
    e("  .amdhsa_user_sgpr_count 2")
    e("  .amdhsa_user_sgpr_kernarg_segment_ptr 1")
    e("  .amdhsa_system_sgpr_workgroup_id_x 1")
    e("  .amdhsa_system_sgpr_workgroup_id_y 0")
    e("  .amdhsa_system_sgpr_workgroup_id_z 0")
    e("  .amdhsa_system_vgpr_workitem_id 0")
    e("  .amdhsa_next_free_vgpr %d" % vgprs)
    e("  .amdhsa_next_free_sgpr 69")
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
      - {.offset: 56, .size: 8, .value_kind: by_value}
      - {.offset: 64, .size: 4, .value_kind: by_value}
    .group_segment_fixed_size: %d
    .kernarg_segment_align: 8
    .kernarg_segment_size: 72
    .max_flat_workgroup_size: %d
    .name: %s
    .private_segment_fixed_size: 0
    .sgpr_count: 76
    .sgpr_spill_count: 0
    .symbol: %s.kd
    .uniform_work_group_size: 1
    .uses_dynamic_stack: false
    .vgpr_count: %d
    .vgpr_spill_count: 0
    .wavefront_size: 64
""" % (LDS_BYTES, threads, name, name, vgprs)
    return "\n".join(o), meta


def generate():
    parts = ['.amdgcn_target "amdgcn-amd-amdhsa--gfx950"', ".amdhsa_code_object_version 6", ""]
    metas = []
    for buckets, waves in VARIANTS:
        text, meta = gen_kernel(buckets, waves)
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
