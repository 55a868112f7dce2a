"""Shows that the pins of the numeric oracle can fail: each case applies one plausible slip to a
copy of ``oracle/monarch_oracle.c`` (a wrong divisor, a rounding per add, a dropped member, a
transposed index chain), builds it, puts it in the oracle's place and expects the named pin test to
fail.  A pin that passes on the mutated build pins nothing."""
import os
import re
import subprocess

import numpy as np
import pytest

import oracle
import test_oracle_collectives as K
import test_oracle_numeric as T
import test_oracle_rdmaxcel as R
import test_oracle_slice as S

SRC = os.path.join(os.path.dirname(oracle.__file__), "monarch_oracle.c")

# (name, function whose body is edited, text to replace, replacement, pin that must fail)
MUTATIONS = [
    ("scatter_bf16_divides_by_n_out", "o_reduce_scatter_bf16", "acc = acc / (float)n_in", "acc = acc / (float)n_out",
     lambda: T.test_reduce_scatter_bf16_member_order(T.AVG, 3, 2)),
    ("scatter_f32_divides_by_n_out", "o_reduce_scatter_f32", "acc = acc / (float)n_in", "acc = acc / (float)n_out",
     lambda: T.test_reduce_scatter_f32_avg_member_order(3, 2)),
    ("scatter_bf16_rounds_per_add", "o_reduce_scatter_bf16", "acc = o_combine_f32(acc, bf16_to_f32(in[g][loc]), op)",
     "acc = bf16_to_f32(f32_to_bf16_rne(acc + bf16_to_f32(in[g][loc])))",
     lambda: T.test_reduce_scatter_bf16_member_order(T.SUM, 5, 4)),
    ("scatter_bf16_drops_last_member", "o_reduce_scatter_bf16", "g < n_in; g++) acc = o_combine_f32(acc, bf16", "g + 1 < n_in; g++) acc = o_combine_f32(acc, bf16",
     lambda: T.test_reduce_scatter_bf16_member_order(T.SUM, 3, 2)),
    ("scatter_f32_skips_in_view", "o_reduce_scatter_f32", "o_slice_get(in_view, i, &loc)", "loc = i",
     lambda: T.test_reduce_scatter_f32_avg_member_order(5, 4)),
    ("f64_accumulates_in_float", "o_reduce_f64", "double acc = in[0][i]", "float acc = (float)in[0][i]",
     lambda: T.test_reduce_f64_left_to_right(3)),
    ("f64_avg_divides_by_n_minus_1", "o_reduce_f64", "acc = acc / (double)n", "acc = acc / (double)(n - 1)",
     lambda: T.test_reduce_f64_left_to_right(3)),
    ("f64_sums_right_to_left", "o_reduce_f64",
     "double acc = in[0][i];\n        for (uint32_t r = 1; r < n; r++) acc += in[r][i];",
     "double acc = in[n - 1][i];\n        for (uint32_t r = n - 1; r-- > 0;) acc += in[r][i];",
     lambda: T.test_reduce_f64_left_to_right(7)),
    ("max_propagates_nan", "o_combine_f32", "case 2: return (x > acc || acc != acc) ? x : acc;",
     "case 2: return (x > acc || x != x) ? x : acc;", K.test_max_min_nan_and_signed_zero_rule),
    ("min_takes_the_later_zero", "o_combine_f32", "case 3: return (x < acc || acc != acc) ? x : acc;",
     "case 3: return (x <= acc || acc != acc) ? x : acc;", K.test_max_min_nan_and_signed_zero_rule),
    ("int8_max_compares_unsigned", "o_reduce_op", "int8_t acc = ((const int8_t*)in[0])[i];\n                for (uint32_t r = 1; r < n; r++) acc = o_combine_i8(acc, ((const int8_t*)in[r])[i], op);",
     "uint8_t acc = ((const uint8_t*)in[0])[i];\n                for (uint32_t r = 1; r < n; r++) acc = o_combine_u8(acc, ((const uint8_t*)in[r])[i], op);",
     lambda: K.test_integer_prod_wraps_and_max_min_follow_the_sign(np.int8)),
    ("bf16_prod_rounds_per_step", "o_reduce_op", "acc = o_combine_f32(acc, bf16_to_f32(((const uint16_t*)in[r])[i]), op);",
     "acc = bf16_to_f32(f32_to_bf16_rne(o_combine_f32(acc, bf16_to_f32(((const uint16_t*)in[r])[i]), op)));",
     lambda: K.test_bf16_and_f16_other_ops_accumulate_in_fp32_and_round_once(K.PROD)),
    ("all_to_all_sends_own_chunk_index", "o_stack_scatter", "(const uint8_t*)in[g] + rank * chunk", "(const uint8_t*)in[g] + g * chunk",
     K.test_stack_scatter_matches_reference_all_to_all_vector),
    ("all_to_all_in_place_reads_overwritten_chunks", "o_stack_scatter",
     "memcpy(tmp + g * chunk, (const uint8_t*)in[g] + rank * chunk, chunk);\n    memcpy(out, tmp, chunk * n);",
     "memcpy((uint8_t*)out + g * chunk, (const uint8_t*)in[(g + 1) % n] + rank * chunk, chunk);\n    for (uint32_t g = 0; g < n; g++) memcpy((uint8_t*)out + g * chunk, (const uint8_t*)in[g] + rank * chunk, chunk);",
     K.test_stack_scatter_matches_reference_all_to_all_vector),
    ("send_route_swaps_the_sides", "o_send_tensor_route", "        *to_rank = peer;", "        *from_rank = peer;",
     K.test_send_tensor_result_is_the_contiguous_view),
    # work-queue / completion-queue entries against the hand-derived bytes
    ("send_wqe_slot_of_48_bytes", "o_send_wqe", "(uint64_t)slot << 6", "(uint64_t)slot * 48",
     lambda: R.test_send_wqe_known_bytes_signaled_write(R.OracleImpl)),
    ("send_wqe_flags_in_the_signature_byte", "o_send_wqe", "wqe[11] = p->signaled", "wqe[8] = p->signaled",
     lambda: R.test_send_wqe_known_bytes_signaled_write(R.OracleImpl)),
    ("send_wqe_lkey_before_byte_count", "o_send_wqe", "put_be32(wqe + 32, (uint32_t)p->length);\n    put_be32(wqe + 36, p->lkey);",
     "put_be32(wqe + 36, (uint32_t)p->length);\n    put_be32(wqe + 32, p->lkey);",
     lambda: R.test_send_wqe_known_bytes_signaled_write(R.OracleImpl)),
    ("send_wqe_data_before_remote_address", "o_send_wqe", "put_be64(wqe + 16, p->raddr);\n    put_be32(wqe + 24, p->rkey);",
     "put_be64(wqe + 40, p->raddr);\n    put_be32(wqe + 24, p->rkey);",
     lambda: R.test_send_wqe_known_bytes_signaled_write(R.OracleImpl)),
    ("send_wqe_record_without_24_bit_mask", "o_send_wqe", "(idx + 1u) & 0xFFFFFFu", "(idx + 1u)",
     lambda: R.test_send_wqe_known_bytes_truncations_and_24_bit_record(R.OracleImpl)),
    ("send_wqe_record_in_the_receive_word", "o_send_wqe", "&p->dbrec[1]", "&p->dbrec[0]",
     lambda: R.test_send_wqe_known_bytes_signaled_write(R.OracleImpl)),
    ("send_wqe_index_not_cut_to_24_bits_by_the_shift", "o_send_wqe", "put_be32(wqe + 0, (idx << 8) | p->op_type);",
     "put_be32(wqe + 0, ((idx & 0xFFFFu) << 8) | p->op_type);",
     lambda: R.test_send_wqe_known_bytes_truncations_and_24_bit_record(R.OracleImpl)),
    ("little_endian_words", "put_be32", "p[0] = (uint8_t)(v >> 24);\n    p[1] = (uint8_t)(v >> 16);\n    p[2] = (uint8_t)(v >> 8);\n    p[3] = (uint8_t)v;",
     "p[3] = (uint8_t)(v >> 24);\n    p[2] = (uint8_t)(v >> 16);\n    p[1] = (uint8_t)(v >> 8);\n    p[0] = (uint8_t)v;",
     lambda: R.test_recv_wqe_known_bytes(R.OracleImpl)),
    ("recv_wqe_record_masked_to_24_bits", "o_recv_wqe", "(uint32_t)(p->wr_id + 1)", "(uint32_t)(p->wr_id + 1) & 0xFFFFFFu",
     lambda: R.test_recv_wqe_known_bytes(R.OracleImpl)),
    ("recv_wqe_record_is_wr_id", "o_recv_wqe", "(uint32_t)(p->wr_id + 1)", "(uint32_t)(p->wr_id)",
     lambda: R.test_recv_wqe_known_bytes(R.OracleImpl)),
    ("cqe_poll_ignores_the_lap", "o_cqe_poll", "((idx / p->cqe_cnt) & 1u)", "0u",
     lambda: R.test_cqe_poll_second_lap_large_entries_and_record_wrap(R.OracleImpl)),
    ("cqe_poll_owns_opcode_15", "o_cqe_poll", " && opcode != 0xF", "",
     lambda: R.test_cqe_poll_known_answers(R.OracleImpl)),
    ("cqe_poll_accepts_opcodes_up_to_7", "o_cqe_poll", "(opcode & 0xC) == 0", "(opcode & 0x8) == 0",
     lambda: R.test_cqe_poll_known_answers(R.OracleImpl)),
    ("cqe_poll_op_own_at_byte_63_of_large_entries", "o_cqe_poll", "cqe[p->cqe_size - 1]", "cqe[63]",
     lambda: R.test_cqe_poll_second_lap_large_entries_and_record_wrap(R.OracleImpl)),
    ("cqe_poll_error_leaves_the_record", "o_cqe_poll", "        *byte_cnt = -2;\n    }", "        *byte_cnt = -2;\n        return;\n    }",
     lambda: R.test_cqe_poll_known_answers(R.OracleImpl)),
    ("db_ring_copies_56_bytes", "o_db_ring", "i < 8", "i < 7",
     lambda: R.test_db_ring_copies_exactly_64_bytes(R.OracleImpl)),
    # Slice algebra
    ("get_peels_the_first_dimension_first", "o_slice_get", "for (uint32_t k = s->ndim; k-- > 0;) {", "for (uint32_t k = 0; k < s->ndim; k++) {",
     lambda: S.test_get_vectors(_vectors())),
    ("get_ignores_the_offset", "o_slice_get", "uint64_t val = s->offset, rest", "uint64_t val = 0, rest",
     lambda: S.test_iter_vectors(_vectors())),      # slice.rs:893-902: {10, [10, 2], [10, 5]} iterates 10, 15, ... and iter == get
    ("new_accepts_overlapping_dimensions", "o_slice_new", "if (total > stride) { rc = O_ERR_STRIDE_TOO_SMALL; break; }", "",
     lambda: S.test_validation_rules()),
    ("new_refuses_equal_strides_of_size_one", "o_slice_new", "stride == prev_stride && size != 1 && prev_size != 1", "stride == prev_stride",
     lambda: S.test_validation_rules()),
    ("location_adds_no_offset", "o_slice_location", "uint64_t v = s->offset;", "uint64_t v = 0;",
     lambda: S.test_len_contiguous_rowmajor()),     # the doc example slice.rs:72-80 and test_at_1d_to_0d, :1031-1043
    ("iter_walks_column_major", "o_slice_iter", "for (uint32_t k = s->ndim; k-- > 0;) {\n            coord[k] = rest % s->sizes[k];",
     "for (uint32_t k = 0; k < s->ndim; k++) {\n            coord[k] = rest % s->sizes[k];", lambda: S.test_iter_vectors(_vectors())),
    ("coordinates_peels_small_strides_first", "o_slice_coordinates", "for (uint32_t r = n; r-- > 0;) {", "for (uint32_t r = 0; r < n; r++) {",
     lambda: S.test_coordinates_index_vectors(_vectors())),
    ("coordinates_accepts_a_remainder", "o_slice_coordinates", "if (pos != 0) return O_ERR_VALUE_NOT_IN_SLICE;", "",
     lambda: S.test_named_and_fuzz_check(_vectors())),   # test_ndslice.py:127-131: no extra elements between the slice's own
    ("index_is_column_major", "o_slice_index", "for (uint32_t k = s->ndim; k-- > 0;) {", "for (uint32_t k = 0; k < s->ndim; k++) {",
     lambda: S.test_coordinates_index_vectors(_vectors())),
    ("select_rounds_the_count_down", "o_slice_select", "(end - begin + step - 1) / step", "(end - begin) / step",
     lambda: S.test_select_at_view_embedding_vectors(_vectors())),
    ("select_keeps_the_stride", "o_slice_select", "out_strides[dim] *= step;", "",
     lambda: S.test_select_at_view_embedding_vectors(_vectors())),
    ("at_keeps_the_offset", "o_slice_at", "*out_offset = s->offset + index * s->strides[dim];", "*out_offset = s->offset;",
     lambda: S.test_select_at_view_embedding_vectors(_vectors())),
    ("subview_checks_starts_only", "o_slice_subview", "starts[d] + lens[d] > s->sizes[d]", "starts[d] >= s->sizes[d]",
     lambda: S.test_subview_inclusion()),
    ("view_accepts_an_offset", "o_slice_view", "if (s->offset != 0) return O_ERR_INCOMPATIBLE_VIEW;", "",
     lambda: S.test_select_at_view_embedding_vectors(_vectors())),
    ("unpack_writes_packed_order", "o_slice_unpack", "(char*)dst_base + loc * elem_size", "(char*)dst_base + i * elem_size",
     lambda: S.test_pack_unpack_against_as_strided()),
    ("pack_runs_all_cores_starts_rows_at_the_offset", "o_pack_runs_mt", "o_slice_get(s, r * run, &loc);", "loc = s->offset + r * run;",
     lambda: S.test_pack_unpack_against_as_strided()),
    ("mesh_members_start_at_the_rank", "o_mesh_dim_members", "uint64_t start = rank - stride * coords[dim];", "uint64_t start = rank;",
     lambda: S.test_device_mesh_vectors(_vectors())),
    ("stack_interleaves_members", "o_stack", "[(uint64_t)g * numel * elem_size + b]", "[(uint64_t)b * n + g]",
     lambda: K.test_stack_matches_reference_all_gather_vector()),
    ("flat_unpack_reads_from_the_start", "o_flat_unpack", "(const char*)flat + offsets[t] * elem_size", "(const char*)flat",
     lambda: T.test_fp8_dequant_accumulate_and_flat()),
    ("f16_subnormals_flush_to_zero", "f32_to_f16_rne", "uint32_t m = (uint32_t)rintf(ldexpf(av, 24));", "uint32_t m = 0;",
     lambda: T.test_f16_round_matches_torch()),
    ("f16_overflow_saturates_instead_of_infinity", "f32_to_f16_rne", "if (e >= 31) return (uint16_t)(sign | 0x7c00u);", "if (e >= 31) return (uint16_t)(sign | 0x7bffu);",
     lambda: T.test_f16_round_matches_torch()),
    ("u8_sum_saturates", "o_reduce_u8", "acc = (uint8_t)(acc + in[r][i]);", "acc = (uint8_t)(acc + in[r][i] > 255 ? 255 : acc + in[r][i]);",
     lambda: T.test_reduce_integer_wraps()),
    # bf16 rounding and the plain reduces
    ("bf16_ties_round_away_from_zero", "f32_to_bf16_rne", "u += 0x7fffu + lsb;", "u += 0x8000u;",
     lambda: T.test_bf16_round_matches_torch()),
    ("bf16_truncates", "f32_to_bf16_rne", "u += 0x7fffu + lsb;", "",
     lambda: T.test_bf16_round_matches_torch()),
    ("bf16_avg_multiplies_by_a_reciprocal", "o_reduce_bf16", "acc = acc / (float)n", "acc = acc * (1.0f / (float)n)",
     lambda: [T.test_reduce_bf16_vs_torch(n) for n in (3, 5, 7)]),
    ("f32_sum_skips_member_one", "o_reduce_f32", "for (uint32_t r = 1; r < n; r++) acc += in[r][i];", "for (uint32_t r = 2; r < n; r++) acc += in[r][i];",
     lambda: T.test_reduce_golden(_vectors())),
    # fp8 codec
    ("e4m3fn_subnormal_grid_of_2_to_minus_10", "o_e4m3fn_encode", "ldexpf(a, 9)", "ldexpf(a, 10)",
     lambda: T.test_e4m3fn_encode_all_bf16_patterns_vs_torch()),
    ("e4m3fn_mantissa_carry_dropped", "o_e4m3fn_encode", "        m = 0;\n        e += 1;", "        m = 7;",
     lambda: T.test_e4m3fn_encode_fp32_ties_and_midpoints()),
    ("e4m3fn_bias_8", "o_e4m3fn_encode", "((e + 7) << 3)", "((e + 8) << 3)",
     lambda: T.test_e4m3fn_encode_all_bf16_patterns_vs_torch()),
    ("e4m3fn_decode_without_subnormals", "o_e4m3fn_decode", "v = ldexpf((float)m, -9);", "v = 0.0f;",
     lambda: T.test_e4m3fn_decode_all_codes_vs_torch()),
    ("quantiser_scales_to_240", "o_fp8_quantize", "float scale = absmax / O_FP8_MAX;", "float scale = absmax / 240.0f;",
     lambda: T.test_fp8_quantize_invariants()),
    ("quantiser_takes_the_max_not_the_absmax", "o_fp8_quantize", "float a = fabsf(bf16_to_f32(x[i]));", "float a = bf16_to_f32(x[i]);",
     lambda: T.test_fp8_quantize_invariants()),
    ("dequantiser_uses_the_next_blocks_scale", "o_fp8_dequant_accumulate", "scales[i / block]", "scales[(i + 1) / block]",
     lambda: T.test_fp8_dequant_accumulate_and_flat()),
]
_VEC = []


def _vectors():
    if not _VEC:
        import json
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ndslice_vectors.json")) as f:
            _VEC.append(json.load(f))
    return _VEC[0]


def _mutate(text, func, old, new):
    # the definition: a line at top level that names the function and opens a body
    start = re.search(r"^[A-Za-z_][\w \*]*\b" + func + r"\([^;{]*\)\s*\{", text, flags=re.M).start()
    end = text.index("\n}\n", start)
    body = text[start:end]
    assert body.count(old) == 1, (func, old, body.count(old))
    return text[:start] + body.replace(old, new) + text[end:]


@pytest.mark.parametrize("name,func,old,new,pin", MUTATIONS, ids=[m[0] for m in MUTATIONS])
def test_pin_fails_on_mutated_oracle(tmp_path, monkeypatch, name, func, old, new, pin):
    with open(SRC) as f:
        text = f.read()
    c = tmp_path / "mutant.c"
    c.write_text(_mutate(text, func, old, new))
    so = tmp_path / "mutant.so"
    subprocess.check_call(["gcc", "-O1", "-fPIC", "-std=c11", "-ffp-contract=off", "-fopenmp", "-shared",
                           "-o", str(so), str(c), "-lm"])
    pin()                                    # green on the real oracle
    monkeypatch.setattr(oracle, "_lib", oracle.load(str(so)))
    try:
        pin()
    except (AssertionError, pytest.fail.Exception, oracle.OracleError):   # a wrong value, an expected error that no longer comes, an error where none belongs
        return
    pytest.fail(f"the pin passes on the mutant {name}: it pins nothing there")
