"""CPU checks of the assembly that gen_eval_reg_kernel.py writes: the copies of tree blocks and border images
from global memory to LDS are followed through the straight-line part of every kernel (up to the tree loop) and
through one turn of the loop, and every source offset and LDS destination must stay inside what the host
allocates. A wrong step of the staging offset faults the GPU; here it fails an assertion."""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _generator():
    path = os.path.join(ROOT, "catboost_amd", "csrc", "gen_eval_reg_kernel.py")
    spec = importlib.util.spec_from_file_location("gen_eval_reg_kernel", path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def _copies(lines, wave, lane, wave_bytes):
    """(source offset from the table's start, LDS address) of every global -> LDS copy of one lane, in order,
    and the index of the first copy of the tree loop."""
    s100 = wave * wave_bytes
    v2 = s28 = m0 = None
    copies, loop_at = [], None
    for line in lines:
        line = line.strip()
        if line.endswith("_loop:") and loop_at is None:
            loop_at = len(copies)
        if line.startswith("v_lshlrev_b32_e32 v2, 2, v1"):
            v2 = lane * 16
        found = re.match(r"s_sub_u32 s28, s100, (\d+)", line)
        if found:
            s28 = (s100 - int(found.group(1))) & 0xffffffff
        if line == "v_add_u32_e32 v2, s28, v2":
            v2 = (v2 + s28) & 0xffffffff
        found = re.match(r"v_add_u32_e32 v2, (0x[0-9a-f]+), v2", line)
        if found:
            v2 = (v2 + int(found.group(1), 16)) & 0xffffffff
        found = re.match(r"s_add_u32 m0, s100, (\d+)", line)
        if found:
            m0 = s100 + int(found.group(1))
        found = re.match(r"global_load_lds_dwordx4 v2, s\[26:27\](?: offset:(\d+))?", line)
        if found:
            offset = int(found.group(1) or 0)
            copies.append(((v2 + offset) & 0xffffffff, m0 + offset + lane * 16))
        if line.startswith("s_branch") and line.endswith("_loop"):
            break
    return copies, loop_at


@pytest.mark.parametrize("fused", [False, True])
def test_staging_copies_stay_inside_the_tables(fused):
    gen = _generator()
    if fused:
        cases = [(buckets, waves, 1, 256, False, six, True, levels) for buckets, waves in gen.FUSED_SHAPES
                 for six in (False, True)
                 for levels in ((None, 6) if buckets <= gen.FUSED_SIX_LEVEL_BUCKETS else (None,))]
    else:
        cases = [variant + (False, None) for variant in gen.VARIANTS]
    for buckets, waves, pitch, leaves, mixed, six, is_fused, levels in cases:
        text, _ = gen.gen_kernel(buckets, waves, pitch, leaves, mixed, six, fused=is_fused, levels=levels)
        lines = text.split("\n")
        block = gen.tree_block(pitch, leaves)
        buf_bytes = block * leaves * pitch * 8
        wave_bytes = buf_bytes // waves
        images = gen.fused_chunks(buckets, six) if is_fused else 0
        name = gen.kernel_name(buckets, waves, pitch, leaves, mixed, six, is_fused)
        for wave, lane in ((0, 0), (waves - 1, 63)):
            copies, loop_at = _copies(lines, wave, lane, wave_bytes)
            assert copies and loop_at is not None, name
            share = wave * wave_bytes + lane * 16
            # before the loop: the border images (fused kernels) and the first tree block, each in whole; in the loop
            # (one turn = two tree blocks) the two blocks behind the one being evaluated
            per_buffer = wave_bytes // 1024
            assert loop_at == (images + 1) * per_buffer, name
            for index, (source, lds) in enumerate(copies):
                assert 0 <= lds and lds + 16 <= 2 * buf_bytes, (name, index, lds)
                # a lane copies the same 16 bytes of its wave's share of a block into the same place of a buffer
                assert lds % buf_bytes == source % buf_bytes == share + (index % per_buffer) * 1024, (name, index, source, lds)
                # the table holds the images, the model's tree blocks and two blocks of null trees behind them;
                # up to the end of the loop's first turn the copies read the images and the first three blocks
                assert source < (images + 3) * buf_bytes, (name, index, source)
                assert source % 16 == 0 and (source % buf_bytes) // wave_bytes == wave, (name, index, source)
            # the blocks are read in order and each lands in the buffer that the kernel evaluates next
            staged = []
            for source, lds in copies:
                item = (source // buf_bytes, lds // buf_bytes)
                if not staged or staged[-1] != item:
                    staged.append(item)
            tail = staged[-3:]
            assert [b for b, _ in tail] == [images, images + 1, images + 2], (name, staged)
            assert [buffer for _, buffer in tail] == [0, 1, 0], (name, staged)
            if is_fused:
                assert [b for b, _ in staged[:images]] == list(range(images)), (name, staged)
                assert [buffer for _, buffer in staged[:images]] == [i % 2 for i in range(images)], (name, staged)
