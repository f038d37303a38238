"""Rows with NaN and infinities for the softmax and LayerNorm tests: the inputs, and what the reference's
arithmetic makes of them (nn_operators/softmax/softmax.h:32-57, nn_operators/layernorm/layernorm.h:13-23).

Softmax: a NaN anywhere, or a +inf (inf - inf), makes every output of the row NaN; -inf elements get
probability exactly 0; a row of nothing but -inf is 0/0 = NaN; -FLT_MAX everywhere is the uniform row.
LayerNorm: a row with a NaN or an infinity has NaN y, mean and rstd.  Rows without special values are
unaffected by their neighbours."""
import numpy as np

FLT_MAX = float(np.finfo(np.float32).max)

# name -> (function filling one row in place, expected class of the row)
#   "nan"     every output NaN
#   "finite"  ordinary parity with the oracle (checked by the caller's tolerance function)
SOFTMAX_ROWS = [
    ("plain", lambda r: None, "finite"),
    ("nan_first", lambda r: r.__setitem__(0, np.nan), "nan"),
    ("nan_middle", lambda r: r.__setitem__(r.size // 2 + 1, np.nan), "nan"),
    ("nan_last", lambda r: r.__setitem__(r.size - 1, np.nan), "nan"),
    ("plus_inf", lambda r: r.__setitem__(3 % r.size, np.inf), "nan"),
    ("two_plus_inf", lambda r: (r.__setitem__(0, np.inf), r.__setitem__(r.size - 1, np.inf)), "nan"),
    ("minus_inf_some", lambda r: r.__setitem__(slice(1, None, 3), -np.inf), "finite"),
    ("minus_inf_all_but_one", lambda r: (r.fill(-np.inf), r.__setitem__(r.size // 3, 2.5)), "finite"),
    ("minus_inf_all", lambda r: r.fill(-np.inf), "nan"),
    ("minus_flt_max_all", lambda r: r.fill(-FLT_MAX), "finite"),
    ("nan_and_inf", lambda r: (r.__setitem__(0, -np.inf), r.__setitem__(1, np.nan), r.__setitem__(2, np.inf)), "nan"),
    ("plain_again", lambda r: None, "finite"),
]

LAYERNORM_ROWS = [
    ("plain", lambda r: None, "finite"),
    ("nan_first", lambda r: r.__setitem__(0, np.nan), "nan"),
    ("nan_middle", lambda r: r.__setitem__(r.size // 2 + 1, np.nan), "nan"),
    ("plus_inf_first", lambda r: r.__setitem__(0, np.inf), "nan"),
    ("plus_inf_last", lambda r: r.__setitem__(r.size - 1, np.inf), "nan"),
    ("minus_inf_middle", lambda r: r.__setitem__(r.size // 2, -np.inf), "nan"),
    ("both_inf", lambda r: (r.__setitem__(1, np.inf), r.__setitem__(r.size - 2, -np.inf)), "nan"),
    ("plain_again", lambda r: None, "finite"),
]


def build(rows_spec, cols, base, repeat=1):
    """[len(rows_spec) * repeat, cols] float32 from `base` rows (shape [n, cols], cycled), each row put through
    its spec; returns (x, classes)."""
    n = len(rows_spec) * repeat
    x = np.array([base[i % base.shape[0]] for i in range(n)], np.float32)
    classes = []
    for i in range(n):
        _, fill, cls = rows_spec[i % len(rows_spec)]
        fill(x[i])
        classes.append(cls)
    return x, np.array(classes)


def check_rows(got, ref, classes, what):
    """NaN rows are NaN everywhere in both; other rows have no NaN in either.  Returns the mask of finite rows."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    nan_rows = classes == "nan"
    if got.ndim == 1:
        got, ref = got[:, None], ref[:, None]
    assert np.all(np.isnan(ref[nan_rows])), "%s: oracle row that should be NaN is not" % what
    assert np.all(np.isnan(got[nan_rows])), "%s: rows %s should be all NaN" % (
        what, np.nonzero(nan_rows & ~np.all(np.isnan(got), axis=1))[0][:8])
    assert not np.any(np.isnan(ref[~nan_rows])), "%s: oracle has NaN in an ordinary row" % what
    assert not np.any(np.isnan(got[~nan_rows])), "%s: NaN in ordinary rows %s" % (
        what, np.nonzero(~nan_rows & np.any(np.isnan(got), axis=1))[0][:8])
    return ~nan_rows
