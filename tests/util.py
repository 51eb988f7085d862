import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rel_err(got, want):
    """Norm-wise relative error of a tensor: max|got - want| / max|want|."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.abs(want).max()
    return np.abs(got - want).max() / (scale if scale > 0 else 1.0)


def assert_close(got, want, tol, what=""):
    assert got.shape == want.shape, "%s: shape %s != %s" % (what, got.shape, want.shape)
    assert np.isfinite(np.asarray(got, dtype=np.float64)).all(), "%s: non-finite values" % what
    e = rel_err(got, want)
    assert e <= tol, "%s: relative error %.3g > %.3g" % (what, e, tol)
    return e


FP32_TOL = 1e-5        # north star: fp32 within 1e-5 relative of the reference path
FP16_TOL = 1e-2        # fp16 storage: 1e-2 relative on pooled / logit outputs (the reference's own fp16-vs-fp32 bound)


def tf_style_fixture():
    """The GraphDef written by google.protobuf from the reference's .proto field numbers
    (tests/golden/make_tf_graphdef_fixture.py): path, {name: tensor a loader must find}, [names it must not]."""
    z = np.load(os.path.join(GOLDEN, "tf_style_graphdef_expected.npz"))
    names = [str(n) for n in z["names"]]
    return (os.path.join(GOLDEN, "tf_style_graphdef.pb"), {n: z["w%03d" % i] for i, n in enumerate(names)},
            [str(n) for n in z["absent"]])
