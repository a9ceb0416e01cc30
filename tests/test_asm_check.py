"""The static check that build.py runs on the assembly of the attention kernels (aeris-gb_amd/asm_check.py), on
hand-written snippets: each rule fires on the pattern it is for and stays quiet on the legal neighbours of that pattern."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("aeris_asm_check", os.path.join(ROOT, "aeris-gb_amd", "asm_check.py"))
asm_check = importlib.util.module_from_spec(spec)
spec.loader.exec_module(asm_check)


def kernel(body):
    return "_ZN5aeris4testEv: ; @test\n" + "\n".join("\t" + l if not l.endswith(":") else l for l in body) + "\n\ts_endpgm\n"


def test_a_read_waited_for_before_its_use_is_fine():
    problems, n = asm_check.check_text(kernel([
        "ds_read_b64_tr_b16 v[10:11], v3 offset:0",
        "ds_read_b64_tr_b16 v[12:13], v3 offset:0x400",
        "v_add_u32_e32 v4, v5, v6",
        "ds_read_b128 v[20:23], v7",             # the compiler's own reads may sit in the window
        "s_waitcnt lgkmcnt(0)",
        "v_mfma_f32_32x32x16_bf16 v[32:47], v[10:13], v[24:27], v[32:47]",
    ]))
    assert n == 2 and problems == []


def test_use_before_the_wait_is_reported():
    problems, _ = asm_check.check_text(kernel([
        "ds_read_b64_tr_b16 v[10:11], v3 offset:0",
        "v_mov_b32_e32 v4, v11",
        "s_waitcnt lgkmcnt(0)",
    ]))
    assert len(problems) == 1 and "before its wait" in problems[0]
    # a wait that does not cover LDS does not end the window
    problems, _ = asm_check.check_text(kernel([
        "ds_read_b64_tr_b16 v[10:11], v3 offset:0",
        "s_waitcnt vmcnt(0)",
        "v_mov_b32_e32 v4, v10",
        "s_waitcnt lgkmcnt(0)",
    ]))
    assert len(problems) == 1


def test_overwriting_a_pending_destination_is_reported():
    problems, _ = asm_check.check_text(kernel([
        "ds_read_b64_tr_b16 v[10:11], v3 offset:0",
        "ds_read_b64_tr_b16 v[11:12], v3 offset:0x400",
        "s_waitcnt lgkmcnt(0)",
    ]))
    assert len(problems) == 1 and "reuses destination" in problems[0]


def test_read_into_the_destination_of_a_running_mfma_is_reported():
    body = ["v_mfma_f32_32x32x16_bf16 v[48:63], v[120:123], v[96:99], v[48:63]",
            "ds_read_b64_tr_b16 v[56:57], v183 offset:0",
            "s_waitcnt lgkmcnt(0)"]
    problems, _ = asm_check.check_text(kernel(body))
    assert len(problems) == 1 and "still writing" in problems[0]
    # far enough behind the MFMA it is legal, and so is a read into the MFMA's SOURCE registers
    far = [body[0]] + ["s_nop 0"] * asm_check.MFMA_WINDOW + body[1:]
    assert asm_check.check_text(kernel(far))[0] == []
    src = [body[0], "ds_read_b64_tr_b16 v[120:121], v183 offset:0", "s_waitcnt lgkmcnt(0)"]
    assert asm_check.check_text(kernel(src))[0] == []


def test_branches_inside_and_into_a_window():
    diamond = ["ds_read_b64_tr_b16 v[10:11], v3 offset:0",
               "s_cbranch_vccnz .LBB0_2",
               "v_add_f32_e32 v20, v21, v22",
               ".LBB0_2:",
               "s_waitcnt lgkmcnt(0)",
               "v_mov_b32_e32 v4, v10"]
    assert asm_check.check_text(kernel(diamond))[0] == []
    # the skipped side of a forward branch is scanned too
    bad_side = list(diamond)
    bad_side[2] = "v_add_f32_e32 v20, v10, v22"
    assert len(asm_check.check_text(kernel(bad_side))[0]) == 1
    # a loop edge from behind the wait back into the window is a second way in
    loop = diamond + ["s_cbranch_scc1 .LBB0_2"]
    problems, _ = asm_check.check_text(kernel(loop))
    assert len(problems) == 1 and "jumps back" in problems[0]


def test_a_read_never_waited_for_is_reported():
    problems, _ = asm_check.check_text(kernel(["ds_read_b64_tr_b16 v[10:11], v3 offset:0"]))
    assert len(problems) == 1 and "not waited for" in problems[0]


def test_state_does_not_leak_between_kernels():
    two = kernel(["ds_read_b64_tr_b16 v[10:11], v3 offset:0", "s_waitcnt lgkmcnt(0)"]) + \
        kernel(["v_mov_b32_e32 v4, v10"]).replace("testEv", "test2Ev")
    assert asm_check.check_text(two) == ([], 1)


def test_counted_wait_behind_stores():
    ok = ["buffer_load_dwordx4 v2, s[44:47], s7 offen lds",
          "global_load_dwordx2 v[8:9], v[4:5], off",
          "global_store_dwordx4 v[40:41], v[20:23], off",
          "global_store_dwordx4 v[40:41], v[4:7], off offset:64",
          "s_waitcnt vmcnt(1)",                       # the compiler's own wait for the load
          "global_store_dwordx4 v[40:41], v[4:7], off offset:96",
          "global_store_dwordx4 v[40:41], v[20:23], off offset:32",
          "s_waitcnt vmcnt(4) lgkmcnt(0)",
          "s_barrier"]
    assert asm_check.check_text(kernel(ok))[0] == []
    # one of the four youngest operations is a load: the wait could leave an LDS load pending
    bad = list(ok)
    bad[2], bad[1] = ok[1], ok[2]
    problems, _ = asm_check.check_text(kernel(bad))
    assert len(problems) == 1 and "not preceded by 4 stores" in problems[0]
    # a label among them: a path could reach the wait without having issued all four
    skip = ok[:6] + [".LBB0_9:"] + ok[6:]
    problems, _ = asm_check.check_text(kernel(skip))
    assert len(problems) == 1 and "not preceded by 4 stores" in problems[0]
    # the main loops' counted waits (no lgkmcnt(0) ... or vmcnt(0)) are not meant
    assert asm_check.check_text(kernel(["buffer_load_dwordx4 v2, s[44:47], s7 offen lds", "s_waitcnt vmcnt(0) lgkmcnt(0)"]))[0] == []
