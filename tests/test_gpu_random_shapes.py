"""Randomized shapes through the bodies of the GPU parity tests: every case is one of the parametrized tests of the other files
called with drawn sizes (row counts around the kernels' dispatch thresholds, widths that end inside blocks and slabs, padded
strides, every layout flag), against the oracle at the same bar as the fixed cases. The draws are seeded: the same cases every run."""
import random

import pytest

import test_gpu_actq as A
import test_gpu_elt as E
import test_gpu_emb as M
import test_gpu_kv as KV
import test_gpu_norm as N
import test_gpu_pfglue as P
import test_gpu_quant as Q
import test_gpu_rope as RP

pytestmark = pytest.mark.gpu


def _generators(r):
    ri, ch = r.randint, r.choice

    def rows():
        return ch([1, 2, 3, 5, 8, 17, 64, 255, 256, 257, 300, 515, 1023, 1024, 1025, 1026, 1030])

    def silu_actq():
        m, f = ri(2, 40), 128 * ri(1, 24)
        return m, f, 2 * f + 4 * ri(0, 8)                      # strides for the wave-per-row form (16-byte rows) and the workgroup form

    def rms_mul():
        wr = ch([1, 1, 2, 4])
        return wr * ri(1, 150), ch([100, 256, 896, 2048, 2560, 3072, 5120, 4 * ri(1, 2000)]), wr

    def qk_nr():
        d, t = ch([64, 96, 128, 256, 512]), ch([1, 3, 16, 400, 600])
        return t, ri(1, 24), d, ch([x for x in (8, 16, 32, 64, 128, 256) if x <= d]), d + 4 * ri(0, 64), ch([1e4, 1e6, 1e7])

    return [
        (A.test_actq_fwd, lambda: (ri(1, 400), 128 * ri(1, 64), ch([1, 3, 7, 7, 7, 15, 127]))),
        (A.test_actq_bwd, lambda: (ri(1, 300), 128 * ri(1, 64), ch([1, 3, 7, 7, 15, 127]))),
        (A.test_block_entry_bwd, lambda: (ri(1, 200), 128 * ri(1, 8), 2 * ri(0, 8))),
        (A.test_block_entry_fwd, lambda: (ri(1, 200), 128 * ch([ri(1, 8), ri(1, 8), ri(9, 64)]), ri(0, 16))),
        (A.test_silu_mul_actq_bwd, silu_actq),
        (A.test_silu_mul_actq_fwd, lambda: (ri(2, 300), 128 * ri(1, 24))),
        (E.test_swiglu, lambda: (ri(1, 70000),)),
        (E.test_silu_mul_bf16, lambda: (ri(1, 300), ri(6, 3000))),
        (E.test_gdn_conv, lambda: (ri(1, 600), ch([6, 64, 100, 256, 512, 1000, 4096, 8200, 10240]))),
        (E.test_gdn_l2, lambda: ch([(ri(1, 1100), ri(1, 48), ch([32, 64, 96, 128, 128, 256])), (ri(1400, 2300), ch([32, 48]), 128)])),
        (E.test_residual_slices_widths, lambda: (ri(1, 400), 4 * ri(1, 700))),
        (M.test_gather_q4k_q80, lambda: (256 * ri(1, 32), ri(4, 2000), ri(3, 600))),
        (M.test_gather_iq4xs_iq2s, lambda: (256 * ri(1, 32), ri(4, 300), ri(3, 300))),
        (M.test_ple_rows_iq4nl, lambda: (ri(1, 100), ri(7, 5000), ri(1, 12))),
        (KV.test_pf_kv_append, lambda: (32 * ri(1, 40), ch([ri(1, 40), ri(1, 40), ri(1024, 1300)]))),
        (KV.test_kv_q8_read_round_trip, lambda: (32 * ri(1, 40), ri(2, 400), ch([False, True]))),
        (N.test_q3p_add_rms16, lambda: (rows(), 256 * ri(1, 8), ri(0, 8), ch([False, True]))),
        (N.test_q35p_add_rms16, lambda: (rows(), 256 * ri(1, 40))),
        (N.test_add_rms_q8_1, lambda: (rows(), 256 * ri(1, 32))),
        (N.test_add_rms_bf16, lambda: (rows(), 256 * ri(1, 32))),
        (N.test_rms_mul_and_rmsnorm, rms_mul),
        (N.test_hc_glue, lambda: (ri(1, 300), ri(1, 4), ch([100, 256, 2048, 2560, 5120, 4 * ri(1, 1500)]))),
        (P.test_gdn_norm, lambda: (ri(1, 5000), 4 * ri(1, 256))),
        (P.test_ple_gate_conv_hist, lambda: (ri(2, 400), ri(1, 4), 32 * ri(1, 24), ri(1, 10))),
        (Q.test_q8_1_plain, lambda: (ri(1, 600000),)),
        (Q.test_mmq_quantize, lambda: (4 * ri(1, 2500), ch([ri(1, 700), ri(1, 700), 2048 + ri(0, 2000)]), ri(0, 1))),
        (Q.test_mmq_quantize_scatter, lambda: (4 * ri(1, 1000), ri(1, 40), ri(1, 8), 4 * ri(0, 3))),
        (Q.test_swiglu_mmq, lambda: (ch([ri(1, 400), ri(1, 400), 2048 + ri(0, 3000)]), ch([4, 8]) * ri(1, 600), 8 * ri(0, 3), ri(0, 1))),
        (RP.test_qk_rope_f16_and_q8, lambda: (ri(1, 96), ri(1, 8), ch([1, 2, 5, 33, 256, 257, 2048, 2051]), ri(0, 120000), ch([False, True]))),
        (RP.test_qk_rope_f16_and_q8, lambda: (4 * ri(1, 10), 4, ch([2048, 2049, 2300]), ri(0, 120000), ch([False, True]))),      # fp32 chunks: whole groups of four heads
        (RP.test_pf_qk_nr, qk_nr),
        (RP.test_qk_rope_bf16, lambda: (ri(1, 96), ri(1, 8), ch([1, 2, 7, 2049]), ri(0, 120000), ch([False, True]), 8 * ri(0, 3))),
    ]


@pytest.mark.parametrize('seed', [20260, 20261])
def test_random_shapes(seed):
    r = random.Random(seed)
    gens = _generators(r)
    for _ in range(250):
        fn, draw = r.choice(gens)
        args = draw()
        try:
            fn(*args)
        except Exception as e:
            raise AssertionError(f'{fn.__module__}.{fn.__name__}{args}: {type(e).__name__}: {e}') from e


def _fused_generators(r):
    import test_gpu_fused_tape as FT
    ri, ch = r.randint, r.choice

    def conv_l2():
        c = 128 * ch([1, 2, 3, 8, 10, 32, 80]); t = ch([ri(1, 40), ri(1, 40), ri(260, 1200), 8192 // (c // 128) + ri(0, 50)])
        return t, c, ri(1, c // 128), ri(0, 1)

    def dense_q8():
        nkv = ri(1, 4)
        return ch([ri(1, 20), ri(1, 20), ri(300, 900)]), ri(1, 24), nkv, ch([16, 32, 64, 128, 256]), ri(0, 3000)

    def qk2():
        d = ch([64, 96, 128, 256, 512])
        return ch([1, 3, 16, 70]), ri(1, 24), ri(1, 4), d, ch([x for x in (8, 16, 32, 64, 128, 256) if x <= d]), ri(0, 1)

    def op_nr():
        d = ch([64, 96, 128, 256, 512])
        return ch([1, 3, 16, 400, 600]), ri(1, 24), d, ch([x for x in (8, 16, 32, 64, 128, 256) if x <= d]), d + 4 * ri(0, 64)

    return [
        (FT.test_gdn_conv_l2_equals_the_two_launches, conv_l2),
        (FT.test_op_gdn_conv_l2_equals_the_two_tape_ops, lambda: (lambda g: (128 * g, ri(1, 20), ri(1, g)))(ch([1, 2, 5, 8, 80]))),
        (FT.test_qk_nr_q8_equals_the_six_launches, dense_q8),
        (FT.test_qk_nr_qk_equals_two_launches, qk2),
        (FT.test_op_qk_nr_reads_its_position_on_the_device, op_nr),
        (FT.test_op_kv_append_three_row_formats, lambda: (32 * ri(1, 40), ch([ri(1, 40), ri(1, 40), ri(1024, 1300)]))),
        (FT.test_op_own_qk_rope_reads_its_position_on_the_device, lambda: (ch([1, 2, 7, 300, 2049, 2100]), ri(0, 1), ri(0, 1))),
        (FT.test_op_own_f16_moe_sum_shexp_add_against_the_oracle,
         lambda: (lambda t: (t * ch([9, 37, 256, 1000, 2048, 5120]), ri(1, 64), t))(ch([1, 2, 3, 16]))),
        (FT.test_qk_nr_kv_equals_the_three_tape_ops,
         lambda: (lambda d: (ch([1, 3, 16, 70]), ri(1, 24), ri(1, 4), d, ch([x for x in (8, 16, 32, 64, 128, 256) if x <= d]), ri(0, 1)))(ch([32, 64, 96, 128, 256, 512]))),
        (FT.test_hadamard_gate_mul16_equals_the_two_tape_ops,
         lambda: (lambda d: (ch([1, 2, 16, 70, 600]), ri(1, 24), d, ch([x for x in (64, 128, 256) if d % x == 0])))(ch([64, 128, 256, 512, 768]))),
    ]


@pytest.mark.parametrize('seed', [30260])
def test_random_shapes_of_the_fused_and_tape_entry_points(seed):
    r = random.Random(seed)
    gens = _fused_generators(r)
    for _ in range(120):
        fn, draw = r.choice(gens)
        args = draw()
        try:
            fn(*args)
        except Exception as e:
            raise AssertionError(f'{fn.__module__}.{fn.__name__}{args}: {type(e).__name__}: {e}') from e
