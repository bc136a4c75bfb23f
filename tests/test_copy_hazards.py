"""The build's scan of the generated GPU code for inline copies that sit too close behind a vector write of one of their
scalar operands (incin_amd/hazards.py): the cases it has to tell apart, on snippets of assembly."""
from incin_amd import hazards

HEAD = "_ZN4test6kernelEv:\n"
COPY = "\t;;#ASMSTART\n\t%s\n\tbuffer_load_dwordx4 v151, s[24:27], s5 offen lds\n\t;;#ASMEND\n"


def test_a_descriptor_restored_right_in_front_of_a_copy_is_reported():
    text = HEAD + "\ts_add_i32 m0, s4, s6\n\tv_readlane_b32 s26, v177, 32\n\tv_readlane_b32 s27, v177, 33\n" + COPY % "s_nop 0"
    found = hazards.scan_asm(text)
    assert len(found) == 1
    func, line, copy, writer, waits = found[0]
    assert func == "_ZN4test6kernelEv" and copy.startswith("buffer_load_dwordx4") and writer.startswith("v_readlane_b32 s27") and waits == 1


def test_five_wait_states_are_enough():
    text = HEAD + "\tv_readlane_b32 s27, v177, 33\n" + COPY % "s_nop 4"
    assert hazards.scan_asm(text) == []
    text = HEAD + "\tv_readlane_b32 s27, v177, 33\n\ts_add_i32 s1, s2, s3\n\ts_add_i32 s1, s2, s3\n\ts_add_i32 s1, s2, s3\n\ts_add_i32 s1, s2, s3\n" + COPY % "s_nop 0"
    assert hazards.scan_asm(text) == []
    text = HEAD + "\tv_readlane_b32 s27, v177, 33\n\ts_add_i32 s1, s2, s3\n\ts_add_i32 s1, s2, s3\n\ts_add_i32 s1, s2, s3\n" + COPY % "s_nop 0"
    assert len(hazards.scan_asm(text)) == 1                     # four


def test_only_the_copys_own_operands_count():
    text = HEAD + "\tv_readlane_b32 s40, v177, 33\n\tv_readfirstlane_b32 s41, v3\n" + COPY % "s_nop 0"
    assert hazards.scan_asm(text) == []
    text = HEAD + "\tv_readfirstlane_b32 s5, v3\n" + COPY % "s_nop 0"              # the scalar offset operand
    assert len(hazards.scan_asm(text)) == 1
    text = HEAD + "\tv_cmp_lt_i32_e64 s[24:25], v1, v2\n" + COPY % "s_nop 0"       # a vector compare into the descriptor's registers
    assert len(hazards.scan_asm(text)) == 1


def test_a_vector_write_of_m0_counts_too():
    text = HEAD + "\tv_readfirstlane_b32 m0, v7\n" + COPY % "s_nop 0"
    assert len(hazards.scan_asm(text)) == 1
    text = HEAD + "\tv_readfirstlane_b32 s9, v7\n\ts_mov_b32 m0, s9\n" + COPY % "s_nop 0"          # through a scalar move: fine
    assert hazards.scan_asm(text) == []


def test_scalar_writes_and_the_second_copy_of_a_group_are_fine():
    text = (HEAD + "\tv_readlane_b32 s27, v177, 33\n" + COPY % "s_nop 4" + "\ts_add_i32 m0, s4, 0x8400\n\ts_mov_b32 s24, s76\n" + COPY % "s_nop 0")
    assert hazards.scan_asm(text) == []


def test_ordinary_loads_are_not_looked_at():
    text = HEAD + "\tv_readlane_b32 s27, v177, 33\n\tbuffer_load_dwordx4 v[0:3], v4, s[24:27], 0 offen\n"
    assert hazards.scan_asm(text) == []          # (the compiler sees those and adds the wait states itself)
