"""The row-program generator without a device: which kernel a program maps to (built in, compiled at run time, or the
interpreter's), the plan it gets, and that the text the generator writes for shapes outside the built-in set compiles
(hipRTC compiles for gfx950 without a GPU).  The addresses are made up: nothing here launches."""
import ctypes as C
import os

import pytest

from axiom_amd import capi

F32, F16, BF16 = capi.DTYPE_F32, capi.DTYPE_F16, capi.DTYPE_BF16


class Prog:
    """A row program over made-up, 256-byte aligned addresses."""

    def __init__(self, rows, cols, dt, out_dt=None, misalign=0):
        self.p = capi.RowsProgram()
        self.p.rows, self.p.cols = rows, cols
        self.p.input, self.p.input_dtype = 0x7F0000000000 + misalign, dt
        self.p.output, self.p.output_dtype = 0x7F1000000000 + misalign, dt if out_dt is None else out_dt
        self.p.norm_weight = self.p.norm_bias = -1
        self.dt, self.post_stage = dt, False

    def _operand(self, kind, dt=None):
        i = self.p.n_operands
        self.p.operands[i].ptr, self.p.operands[i].dtype, self.p.operands[i].kind = 0x7F2000000000 + (i << 32), self.dt if dt is None else dt, capi.BK[kind]
        self.p.n_operands = i + 1
        return i

    def op(self, name, kind=None, imm=None, dt=None):
        chain, n = (self.p.post, self.p.n_post) if self.post_stage else (self.p.pre, self.p.n_pre)
        chain[n].op = capi.OP[name]
        chain[n].operand = -1 if kind is None else self._operand(kind, dt)
        if imm is not None:
            chain[n].imm, chain[n].imm_kind = imm, capi.BK["imm"]
        if self.post_stage:
            self.p.n_post = n + 1
        else:
            self.p.n_pre = n + 1
        return self

    def row(self, name, affine=0):
        self.p.row_op, self.p.eps, self.post_stage = capi.ROWOP[name], 1e-5, True
        if affine >= 1:
            self.p.norm_weight = self._operand("rowvec")
        if affine >= 2:
            self.p.norm_bias = self._operand("rowvec")
        return self

    def reduce(self, name):
        self.p.reduce = capi.RED[name]
        return self

    def name(self):
        return capi.lib().axhip_fused_rows_kernel_name(C.byref(self.p)).decode()

    def prepare(self):
        lib = capi.lib()
        rc = lib.axhip_fused_rows_prepare(C.byref(self.p))
        return rc, (lib.axhip_last_error() or b"").decode()


def test_known_patterns_map_to_built_in_kernels():
    assert Prog(16384, 4096, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it8"
    assert Prog(16384, 4096, BF16).row("layernorm", 2).op("gelu").name() == "rows_static_layernorm_gelu_wb_bf16_g64_it8"
    assert Prog(16384, 4096, BF16).row("rmsnorm", 1).op("gelu").name() == "rows_static_rmsnorm_gelu_w_bf16_g64_it8"
    assert Prog(8192, 8192, F32).op("relu").op("add", imm=1.0).op("mul", "full").row("softmax").reduce("sum").name() == \
        "rows_static_relu_adds_mulf_softmax_sum_f32_g256_it8"
    assert Prog(30000, 1500, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it3_grid"  # 1500 * 2 bytes: rows not 16-byte aligned
    assert Prog(64, 1024, BF16).op("add", "full").row("layernorm", 2).name() == "rows_static_addf_layernorm_wb_bf16_g64_it2"
    assert Prog(64, 1024, F16).op("add", "full").row("layernorm", 2).name() == "rows_jit_addf_layernorm_wb_f16_g64_it2"  # f16 shapes are compiled on first use


def test_other_shapes_are_compiled_at_run_time_and_named_after_their_chain():
    assert Prog(4096, 4096, BF16).row("layernorm", 2).op("sigmoid").name() == "rows_jit_layernorm_sigmoid_wb_bf16_g64_it8"
    assert Prog(4096, 4096, BF16).op("mul", imm=0.5).op("tanh").op("add", "full").row("softmax").name() == "rows_jit_muls_tanh_addf_softmax_bf16_g64_it8"
    # a built-in kernel whose plan has at most 1.15 times the chunk slots of the tightest one serves (8 chunks per lane for 7) ...
    assert Prog(128, 3584, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it8"
    # ... beyond that the tight plan is compiled: a wavefront row of 9 or 10 chunks per lane instead of a 256-thread
    # block with a third of it idle
    assert Prog(128, 4104, BF16).row("layernorm", 2).name() == "rows_jit_layernorm_wb_bf16_g64_it9"
    assert Prog(128, 5000, BF16).row("rmsnorm", 1).name() == "rows_jit_rmsnorm_w_bf16_g64_it10"
    # softmax holds the row as fp32 as well (2 waves per SIMD then): still ahead of the 256-thread block, 50.7 against 53.4 us
    # on [16384, 5000]; so is a row of two streams (layer norm of x + y over 4099 columns: 72 against 95 us)
    assert Prog(128, 5000, BF16).row("softmax").name() == "rows_jit_softmax_bf16_g64_it10"
    assert Prog(128, 4099, BF16).op("add", "full").row("layernorm", 2).name() == "rows_jit_addf_layernorm_wb_bf16_g64_it9_ragged"
    # three 16-bit streams no longer fit
    assert Prog(128, 4104, BF16).op("add", "full").op("mul", "full").row("softmax").name().endswith("_g256_it3")


def test_chunks_are_16_bytes_of_the_widest_full_size_stream():
    # 16-bit in, 16-bit out: 8 elements per chunk -> 4096 columns are 512 chunks, 8 per lane of a wavefront
    assert Prog(1024, 4096, BF16).row("rmsnorm", 1).name().endswith("_bf16_g64_it8")
    # fp32 output: 4 elements per chunk -> 1024 chunks, 4 per thread of a 256-thread block; the label names the result type
    assert Prog(1024, 4096, BF16, out_dt=F32).row("rmsnorm", 1).name() == "rows_jit_rmsnorm_w_bf16_to_f32_g256_it4"
    # an fp32 full-size operand: the same
    assert Prog(1024, 4096, BF16).op("add", "full", dt=F32).row("softmax").name().endswith("_g256_it4")
    # an fp32 per-column operand does not change the chunk: it is read from cache, not streamed
    assert Prog(1024, 4096, BF16).op("mul", "rowvec", dt=F32).row("softmax").name().endswith("_g64_it8")
    # a reduced output ([rows] values) has no chunks
    assert Prog(1024, 4096, BF16, out_dt=F32).op("square").reduce("mean").name().endswith("_bf16_g64_it8")


def test_long_rows_get_a_1024_thread_block_and_beyond_8_chunks_per_thread_stay_as_raw_words():
    # up to 8192 chunks: held as fp32 like the shorter rows
    assert Prog(64, 50304, BF16).row("softmax").name() == "rows_jit_softmax_bf16_g1024_it7"
    assert Prog(64, 32768, F32).row("logsoftmax").name() == "rows_jit_logsoftmax_f32_g1024_it8"
    # 8193 to 16384 chunks: the raw words stay, every pass unpacks them again (a vocabulary of 128 256 16-bit logits)
    assert Prog(64, 128256, BF16).row("softmax").name() == "rows_jit_softmax_bf16_g1024_it16"
    assert Prog(64, 50304, F32).row("layernorm", 2).name() == "rows_jit_layernorm_wb_f32_g1024_it13"
    assert Prog(64, 50257, F32).op("mul", imm=0.5).row("softmax").name() == "rows_jit_muls_softmax_f32_g1024_it13_grid"
    # two 16-bit streams fit up to 9 chunks each per thread, not 16
    assert Prog(64, 70000, BF16).op("add", "full").row("softmax").name() == "rows_jit_addf_softmax_bf16_g1024_it9"
    # beyond that (aligned rows): the block walks the row in steps of 4 chunks per thread, once per pass
    assert Prog(64, 128256, BF16).op("add", "full").row("softmax").name() == "rows_jit_addf_softmax_bf16_g1024_it4_loop"
    assert Prog(64, 128256, F32).row("softmax").name() == "rows_jit_softmax_f32_g1024_it4_loop"
    assert Prog(4, 1 << 20, BF16).row("layernorm", 2).op("gelu").name() == "rows_jit_layernorm_gelu_wb_bf16_g1024_it4_loop"
    assert Prog(4, 200000, F32).op("abs").reduce("max").name() == "rows_jit_abs_reduce_max_f32_g1024_it4_loop"


def test_ragged_rows_take_the_grid_form_when_every_stream_is_full_size_and_equally_aligned():
    """Rows whose length the 16-byte chunk does not divide.  Chunks on memory's 16-byte grid ("_grid": aligned accesses,
    a masked partial chunk at either end of the row) need the input, the full-size operands and the output at one
    address modulo 16, no per-column operand, and more than two chunks per lane; everything else is addressed from
    the row's start ("_ragged": every access unaligned)."""
    assert Prog(4096, 4099, BF16).row("softmax").name() == "rows_jit_softmax_bf16_g64_it9_grid"
    assert Prog(4096, 4099, BF16, misalign=6).row("softmax").name() == "rows_jit_softmax_bf16_g64_it9_grid"  # input and output shifted alike
    assert Prog(4096, 1500, BF16).op("add", "full").row("softmax").name() == "rows_jit_addf_softmax_bf16_g64_it3_grid"  # (built in for the main plans only: 1, 2, 4, 8 chunks per lane)
    assert Prog(4096, 4099, BF16, out_dt=F32).op("square").reduce("sum").name() == "rows_jit_square_reduce_sum_bf16_g64_it9_grid"  # [rows] results: any alignment
    # a per-column operand: its position in the row does not follow the grid
    assert Prog(4096, 1500, BF16).row("layernorm", 2).name() == "rows_static_layernorm_wb_bf16_g64_it3_ragged"
    assert Prog(4096, 1500, BF16).op("mul", "rowvec").row("softmax").name().endswith("_it3_ragged")
    assert Prog(4096, 1500, BF16).row("layernorm").name() == "rows_jit_layernorm_bf16_g64_it3_grid"  # no weight, no bias
    assert Prog(4096, 4099, F32).row("layernorm", 2).name() == "rows_jit_layernorm_wb_f32_g256_it5_ragged"
    # ... but for 1024-thread rows, whose unaligned form would spill
    assert Prog(64, 50257, F32).row("layernorm", 2).name() == "rows_jit_layernorm_wb_f32_g1024_it13_grid"
    # at most two chunks per lane: the extra chunk of the grid form costs more than its aligned accesses gain
    assert Prog(4096, 1001, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it2_ragged"
    # streams at different addresses modulo 16
    p = Prog(4096, 1500, BF16).op("add", "full").row("softmax")
    p.p.operands[0].ptr += 2
    assert p.name().endswith("_it3_ragged")
    p = Prog(4096, 1500, BF16).row("softmax")
    p.p.output += 4
    assert p.name().endswith("_it3_ragged")
    # rows of 16-byte multiples from a base that is not: one shift for every row, still the grid
    assert Prog(4096, 4096, BF16, misalign=2).row("softmax").name() == "rows_jit_softmax_bf16_g64_it9_grid"


def test_short_aligned_rows_share_a_wavefront():
    """Up to 32 chunks (256 16-bit or 128 fp32 columns): 4, 8, 16 or 32 lanes per row, one chunk each, several rows to
    a wavefront; built in like the longer plans.  Odd lengths keep a wavefront per row."""
    assert Prog(1 << 20, 64, BF16).row("softmax").name() == "rows_static_softmax_bf16_g8_it1"
    assert Prog(1 << 20, 16, BF16).row("rmsnorm", 1).name() == "rows_static_rmsnorm_w_bf16_g4_it1"
    assert Prog(1 << 20, 128, BF16).row("layernorm", 2).op("gelu").name() == "rows_static_layernorm_gelu_wb_bf16_g16_it1"
    assert Prog(1 << 20, 128, F32).row("softmax").name() == "rows_static_softmax_f32_g32_it1"
    assert Prog(1 << 20, 100, F32).row("softmax").name() == "rows_static_softmax_f32_g32_it1"  # 25 chunks: seven idle lanes per row
    assert Prog(1 << 20, 256, BF16).op("square").reduce("mean").name() == "rows_static_square_reduce_sum_bf16_g32_it1"
    assert Prog(1 << 20, 264, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it1"  # 33 chunks
    # odd lengths: the same on memory's 16-byte grid, a masked partial chunk at either end of every row
    assert Prog(1 << 14, 77, BF16).row("softmax").name() == "rows_static_softmax_bf16_g16_it1_grid"
    assert Prog(1 << 14, 10, F32).row("logsoftmax").name() == "rows_jit_logsoftmax_f32_g4_it1_grid"
    assert Prog(1 << 14, 5, BF16).row("softmax").name() == "rows_static_softmax_bf16_g4_it1_grid"  # shorter than a chunk
    assert Prog(1 << 14, 197, BF16).row("layernorm", 2).name() == "rows_static_layernorm_wb_bf16_g32_it1_grid"
    assert Prog(1 << 14, 250, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it1_ragged"  # 33 chunks on the grid
    p = Prog(1 << 20, 77, BF16).row("softmax")
    p.p.output += 2  # input and output at different addresses modulo 16: a wavefront per row, from the row's first element
    assert p.name() == "rows_static_softmax_bf16_g64_it1_ragged"
    assert Prog(1 << 20, 96, BF16).op("mul", "colvec").op("tanh").row("softmax").name() == "rows_jit_mulc_tanh_softmax_bf16_g16_it1"


def test_many_short_rows_of_odd_length_go_through_lds():
    """From 32768 rows on: 64 / L consecutive rows per wavefront staged in LDS, L lanes per row (as few as keep a
    lane's share of the row at 64 values or fewer), up to 96 values per lane; the label gives L, the LDS KiB per
    wavefront and stream, and the chunks per lane.  The streams may differ in element size."""
    assert Prog(1 << 20, 77, BF16).row("softmax").name() == "rows_jit_softmax_bf16_lane2_5k_it5"
    assert Prog(1 << 20, 10, F32).row("logsoftmax").name() == "rows_jit_logsoftmax_f32_lane1_3k_it3"
    assert Prog(1 << 20, 5, BF16).row("softmax").name() == "rows_jit_softmax_bf16_lane1_1k_it1"
    assert Prog(1 << 20, 197, BF16).row("layernorm", 2).name() == "rows_jit_layernorm_wb_bf16_lane4_7k_it7"
    assert Prog(1 << 20, 250, BF16).row("softmax").name() == "rows_jit_softmax_bf16_lane4_8k_it8"
    assert Prog(1 << 20, 513, BF16).row("softmax").name() == "rows_jit_softmax_bf16_lane8_9k_it9"
    assert Prog(1 << 20, 1001, BF16).row("softmax").name() == "rows_static_softmax_bf16_g64_it2_ragged"  # 128 values per lane: a wavefront per row
    assert Prog(1 << 20, 77, BF16, out_dt=F32).op("mul", "full").row("rmsnorm", 1).name() == "rows_jit_mulf_rmsnorm_w_bf16_to_f32_lane2_10k_it10"
    assert Prog(1 << 20, 77, BF16, misalign=2).row("softmax").name().endswith("_g16_it1_grid")  # the arrays must start on a 16-byte boundary
    assert Prog((1 << 15) - 1, 77, BF16).row("softmax").name() == "rows_static_softmax_bf16_g16_it1_grid"


def test_large_elementwise_chains_run_as_row_programs_without_a_row_operation():
    """From 8 MiB on, a chain with no row operation and no reduction takes a compiled kernel too.  Where its operands are
    full-size arrays, one-element arrays or immediates the array is seen as rows of 512 chunks whatever its shape; a
    per-column or per-row operand keeps the shape (aligned rows of up to 2048 chunks)."""
    assert Prog(1024, 4096, F32).op("relu").op("mul", "full").name() == "rows_jit_relu_mulf_map_f32_g64_it8"
    assert Prog(1, 1 << 26, BF16).op("gelu").name() == "rows_jit_gelu_map_bf16_g64_it8"  # a vector: 16384 rows of 4096
    assert Prog(1 << 20, 64, BF16).op("mul", imm=0.5).op("add", "scalar").name() == "rows_jit_muls_adds_map_bf16_g64_it8"
    assert Prog(16384, 1024, BF16).op("add", "rowvec").op("relu").name() == "rows_jit_addr_relu_map_bf16_g64_it2"  # a bias: by column
    assert Prog(1 << 20, 64, BF16).op("mul", "colvec").name() == "rows_jit_mulc_map_bf16_g8_it1"
    assert Prog(16384, 4100, BF16).op("add", "rowvec").name().startswith("elementwise_")  # rows that are not whole 16-byte vectors
    assert Prog(4099, 4099, BF16).op("relu").name().startswith("elementwise_")  # no whole number of 4096-element rows
    assert Prog(16384, 4096, BF16, misalign=2).op("relu").name().startswith("elementwise")
    assert Prog(16384, 4096, BF16, out_dt=F32).op("relu").name() == "rows_jit_relu_map_bf16_to_f32_g64_it8"  # fp32 out: rows of 2048
    assert Prog(16384, 4096, BF16, out_dt=capi.DTYPE_U8).op("gt", "full").name() == "rows_jit_gtf_map_bf16_to_u8_g64_it8"  # a comparison's truth values


def test_what_the_compiled_form_does_not_take_goes_to_the_interpreter():
    assert Prog(256, 4096, F32).op("relu").op("mul", "full").name() == "elementwise_e4"  # no row op, no reduction, under 8 MiB
    assert Prog(4, 1000001, BF16).row("softmax").name() == "rows_streamed_e1"  # beyond 16384 chunks and not whole vectors
    # ragged rows whose streams differ in element size
    assert Prog(64, 1001, BF16, out_dt=F32).row("softmax").name().startswith("rows_resident_")


@pytest.mark.parametrize("build", [
    lambda: Prog(4096, 4096, BF16).row("layernorm", 2).op("sigmoid"),
    lambda: Prog(4096, 4096, BF16, out_dt=F32).row("rmsnorm", 1).op("mul", "full"),
    lambda: Prog(4096, 4099, F16).op("abs").op("mul", "full").row("softmax"),
    lambda: Prog(4096, 12000, F32).op("mul", "colvec").op("add", "scalar").row("logsoftmax").op("exp"),
    lambda: Prog(4096, 5000, BF16).op("relu").op("max", imm=0.25).reduce("max"),
    lambda: Prog(64, 128256, F16).op("mul", imm=0.5).row("logsoftmax"),
    lambda: Prog(64, 128256, F32).op("mul", "rowvec").op("add", "full").row("logsoftmax").op("exp").reduce("sum"),
    lambda: Prog(1 << 16, 96, BF16).op("mul", "colvec").op("add", "rowvec").row("layernorm", 2).op("silu"),
    lambda: Prog(1 << 16, 197, F16, out_dt=F32).op("mul", "colvec").op("add", "rowvec").op("sub", "full").row("layernorm", 2).op("silu"),
    lambda: Prog(1 << 16, 45, F32).op("abs").reduce("mean"),
    lambda: Prog(16384, 4096, BF16).op("mul", "full").op("add", "rowvec").op("silu"),
], ids=["post_activation", "gated_norm_fp32_out", "ragged_two_streams", "block_512_with_row_and_scalar_operands", "reduction_it10", "raw_resident_it16",
        "looped_row", "short_rows_16_lanes", "lds_rows_three_spans", "lds_rows_reduction", "elementwise_chain"])
def test_generated_kernels_compile(build):
    prog = build()
    assert prog.name().startswith("rows_jit_"), prog.name()
    rc, err = prog.prepare()
    assert rc == 0, err


def test_run_time_compilation_can_be_switched_off():
    prog = Prog(128, 4104, BF16).row("layernorm", 2)
    assert prog.name() == "rows_jit_layernorm_wb_bf16_g64_it9"
    os.environ["AXHIP_JIT"] = "0"  # read at every dispatch
    try:
        assert prog.name() == "rows_static_layernorm_wb_bf16_g256_it3"  # the built-in kernel of the next looser plan
        assert Prog(128, 4096, BF16).row("layernorm", 2).op("sigmoid").name().startswith("rows_resident_")  # no built-in kernel: the interpreter
    finally:
        del os.environ["AXHIP_JIT"]
