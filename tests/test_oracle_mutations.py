"""Shows that the pins of the numeric oracle can fail: each case applies one plausible slip to a
copy of ``oracle/monarch_oracle.c`` (a wrong divisor, a rounding per add, a dropped member, a
transposed index chain), builds it, puts it in the oracle's place and expects the named pin test to
fail.  A pin that passes on the mutated build pins nothing."""
import os
import subprocess

import pytest

import oracle
import test_oracle_numeric as T

SRC = os.path.join(os.path.dirname(oracle.__file__), "monarch_oracle.c")

# (name, function whose body is edited, text to replace, replacement, pin that must fail)
MUTATIONS = [
    ("scatter_bf16_divides_by_n_out", "o_reduce_scatter_bf16", "acc = acc / (float)n_in", "acc = acc / (float)n_out",
     lambda: T.test_reduce_scatter_bf16_member_order(T.AVG, 3, 2)),
    ("scatter_f32_divides_by_n_out", "o_reduce_scatter_f32", "acc = acc / (float)n_in", "acc = acc / (float)n_out",
     lambda: T.test_reduce_scatter_f32_avg_member_order(3, 2)),
    ("scatter_bf16_rounds_per_add", "o_reduce_scatter_bf16", "acc += bf16_to_f32(in[g][loc])",
     "acc = bf16_to_f32(f32_to_bf16_rne(acc + bf16_to_f32(in[g][loc])))",
     lambda: T.test_reduce_scatter_bf16_member_order(T.SUM, 5, 4)),
    ("scatter_bf16_drops_last_member", "o_reduce_scatter_bf16", "g < n_in; g++) acc += bf16", "g + 1 < n_in; g++) acc += bf16",
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
]


def _mutate(text, func, old, new):
    start = text.index(func + "(")
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
    with pytest.raises(AssertionError):
        pin()
