"""The reference's fresh init (`init_params`, ojas-model/src/init.rs:15-114): the oracle's
restatement pinned by what the reference's own tests and the mathematics fix, then the product's
host routine held to it bit for bit. No device involved."""
import ctypes as C
import math
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "oracle"))
import init_exact as ie  # noqa: E402

NATIVE = ROOT / "ojas_amd" / "libojas_nanolab.so"


def test_fnv1a_matches_the_published_vectors():
    # ojas-model/src/init.rs:127-133
    assert ie.fnv1a(b"") == 0xCBF29CE484222325
    assert ie.fnv1a(b"a") == 0xAF63DC4C8601EC8C
    assert ie.fnv1a(b"foobar") == 0x85944171F73967E8


def test_counter_rng_is_the_pinned_splitmix64_stream():
    # ojas-data/src/rng.rs:58-66
    r = ie.CounterRng(0)
    assert [r.next_u64() for _ in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    top = ie.CounterRng((1 << 64) - 1)
    assert top.next_u64() == 0xE4D971771B652C20
    assert top.state == 0x9E3779B97F4A7C14


def test_zeros_and_ones_are_exact_and_ignore_the_seed():
    for seed in (0, 7, (1 << 64) - 1):
        z = ie.init_values("blocks.0.mixer.o_proj.weight", 33, ie.ZEROS, seed)
        o = ie.init_values("norm_f.weight", 33, ie.ONES, seed)
        assert z.dtype == np.float32 and not z.view(np.uint32).any()  # +0.0, not -0.0
        assert (o.view(np.uint32) == 0x3F800000).all()


def test_box_muller_pairs_obey_the_identities_the_method_fixes():
    """From the raw draws of the same stream: z0^2 + z1^2 = -2 ln u1 and atan2(z1, z0) = 2 pi u2
    (so the cosine branch comes first and the angle uses the second draw), with u1 in (0, 1]."""
    seed = 0x1234
    raw = ie.CounterRng(seed)
    z = ie.normal_stream(seed)
    for _ in range(2000):
        a, b = raw.next_u64(), raw.next_u64()
        u1 = ((a >> 11) + 1) / 2.0 ** 53
        u2 = (b >> 11) / 2.0 ** 53
        assert 0.0 < u1 <= 1.0 and 0.0 <= u2 < 1.0
        z0, z1 = next(z), next(z)
        assert math.isclose(z0 * z0 + z1 * z1, -2.0 * math.log(u1), rel_tol=1e-12, abs_tol=1e-300)
        angle = math.atan2(z1, z0) % math.tau
        assert abs(angle - math.tau * u2) < 1e-9 or abs(angle - math.tau * u2) > math.tau - 1e-9


def test_the_first_draw_can_reach_one_but_never_zero():
    # (x >> 11) + 1 over 2^53: the largest draw gives u1 = 1 (ln = 0, z = 0), the smallest 2^-53.
    assert float((((1 << 64) - 1) >> 11) + 1) / 2.0 ** 53 == 1.0
    assert float((0 >> 11) + 1) / 2.0 ** 53 == 2.0 ** -53
    assert math.isfinite(math.sqrt(-2.0 * math.log(2.0 ** -53)))


def test_normal_values_have_the_moments_of_n_0_std():
    v = ie.init_values("tok_emb.weight", 200_000, ie.NORMAL, 42).astype(np.float64)
    std = float(np.float32(0.02))
    n = v.size
    assert abs(v.mean()) < 5 * std / math.sqrt(n)
    assert abs(v.std() / std - 1.0) < 5 / math.sqrt(2 * n)
    kurt = ((v - v.mean()) ** 4).mean() / v.var() ** 2
    assert abs(kurt - 3.0) < 5 * math.sqrt(24 / n)
    skew = ((v - v.mean()) ** 3).mean() / v.std() ** 3
    assert abs(skew) < 5 * math.sqrt(6 / n)
    # Successive values (a pair's two branches, and neighbours across pairs) are uncorrelated.
    for lag in (1, 2, 3):
        assert abs(np.corrcoef(v[:-lag], v[lag:])[0, 1]) < 5 / math.sqrt(n)


def test_a_value_is_std_times_z_rounded_once():
    seed, name = 9, "blocks.3.ffn.up.weight"
    z = ie.normal_stream(seed ^ ie.fnv1a(name.encode()))
    want = np.array([float(np.float32(0.02)) * next(z) for _ in range(64)]).astype(np.float32)
    got = ie.init_values(name, 64, ie.NORMAL, seed)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    # The f32 constant widened (0.0199999995...), not the decimal 0.02: over many values the two
    # round to different f32 bits somewhere.
    assert ie.INIT_STD_F32 == float(np.float32(0.02)) != 0.02
    z = ie.normal_stream(seed ^ ie.fnv1a(name.encode()))
    decimal = np.array([0.02 * next(z) for _ in range(4096)]).astype(np.float32)
    assert (decimal.view(np.uint32) != ie.init_values(name, 4096, ie.NORMAL, seed).view(np.uint32)).any()


def test_streams_depend_on_name_and_seed_only():
    a = ie.init_values("blocks.0.mixer.q_proj.weight", 4096, ie.NORMAL, 5)
    b = ie.init_values("blocks.0.mixer.k_proj.weight", 4096, ie.NORMAL, 5)
    c = ie.init_values("blocks.0.mixer.q_proj.weight", 4096, ie.NORMAL, 6)
    again = ie.init_values("blocks.0.mixer.q_proj.weight", 4096, ie.NORMAL, 5)
    assert (a.view(np.uint32) == again.view(np.uint32)).all()
    for other in (b, c):
        assert abs(np.corrcoef(a, other)[0, 1]) < 0.08  # 5 / sqrt(4096)
        assert (a != other).mean() > 0.99
    # A longer draw of the same parameter extends the shorter one.
    longer = ie.init_values("blocks.0.mixer.q_proj.weight", 5000, ie.NORMAL, 5)
    assert (longer[:4096].view(np.uint32) == a.view(np.uint32)).all()


def test_param_table_has_the_reference_order_names_and_rules():
    rows = ie.param_table(2, 64, 4, 2, 16, 96, 128)
    assert len(rows) == 2 + 14 * 2  # names.rs:161
    assert rows[0] == ("tok_emb.weight", (128, 64), ie.NORMAL) and rows[-1] == ("norm_f.weight", (64,), ie.ONES)
    by = {n: (s, i) for n, s, i in rows}
    # names.rs:324-340 (each field's name), :236-243 and :290-296 (the zero-initialised outputs)
    assert by["blocks.1.mixer.o_proj.weight"] == ((64, 64), ie.ZEROS)
    assert by["blocks.1.ffn.down.weight"] == ((64, 96), ie.ZEROS)
    assert by["blocks.1.mixer.k_proj.weight"] == ((32, 64), ie.NORMAL)
    assert by["blocks.0.mixer.gate.weight"] == ((4, 64), ie.NORMAL)
    assert by["blocks.0.mixer.gate.bias"] == ((4,), ie.ZEROS)
    assert by["blocks.0.mixer.vr_lambda"] == ((1,), ie.ZEROS)
    assert by["blocks.0.mixer.q_norm.weight"] == ((16,), ie.ONES)
    assert [n for n, _, _ in rows[1:15]] == [f"blocks.0.{x}" for x in (
        "norm1.weight", "mixer.q_proj.weight", "mixer.k_proj.weight", "mixer.v_proj.weight", "mixer.o_proj.weight",
        "mixer.q_norm.weight", "mixer.k_norm.weight", "mixer.gate.weight", "mixer.gate.bias", "mixer.vr_lambda",
        "norm2.weight", "ffn.gate.weight", "ffn.up.weight", "ffn.down.weight")]


# ---- the product's host routine against the oracle -------------------------------------------

@pytest.fixture(scope="module")
def native():
    if not NATIVE.exists():
        pytest.fail(f"{NATIVE} is not built; run __graft_entry__.build()")
    lib = C.CDLL(str(NATIVE))
    lib.onano_fnv1a.restype = C.c_uint64
    lib.onano_fnv1a.argtypes = [C.c_char_p, C.c_uint64]
    lib.onano_reference_init_values.argtypes = [C.c_char_p, C.c_uint64, C.c_int32, C.c_float, C.c_uint64, C.c_void_p]
    return lib


def test_product_fnv1a_equals_the_published_vectors(native):
    assert native.onano_fnv1a(b"", 0) == 0xCBF29CE484222325
    assert native.onano_fnv1a(b"a", 1) == 0xAF63DC4C8601EC8C
    assert native.onano_fnv1a(b"foobar", 6) == 0x85944171F73967E8


@pytest.mark.parametrize("seed", [0, 1, 0xDEADBEEFCAFEF00D, (1 << 64) - 1])
def test_product_init_values_equal_the_oracle_bit_for_bit(native, seed):
    for name, shape, init in ie.param_table(2, 64, 4, 2, 16, 96, 128):
        n = int(np.prod(shape))
        got = np.full(n, np.nan, np.float32)
        rc = native.onano_reference_init_values(name.encode(), n, init, np.float32(0.02), seed, got.ctypes.data_as(C.c_void_p))
        assert rc == 0
        want = ie.init_values(name, n, init, seed)
        assert (got.view(np.uint32) == want.view(np.uint32)).all(), name


def test_product_refuses_a_bad_std(native):
    # init.rs:136-145
    out = np.zeros(4, np.float32)
    for std in (0.0, -0.02, float("nan"), float("inf")):
        rc = native.onano_reference_init_values(b"w", 4, ie.NORMAL, np.float32(std), 1, out.ctypes.data_as(C.c_void_p))
        assert rc == 3, std  # OMX_OUT_OF_RANGE
    assert native.onano_reference_init_values(b"w", 4, 9, np.float32(0.02), 1, out.ctypes.data_as(C.c_void_p)) == 3
