"""The rules by which the kernel wrappers choose workgroup shapes and split counts were measured at a few models'
sizes; between and beyond those they choose speed, not results, but what they return must always be something the
kernels take.  Checked here over a grid of sizes, on the CPU (the rules are plain functions of the sizes)."""
import itertools

from easy_gpt.cpp_amd.kernels.hip import HipKernels as K

BATCHES = [1, 2, 3, 7, 8, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 128, 200, 256, 257, 512, 1000, 4096]
CONTEXTS = [1, 15, 16, 33, 64, 100, 511, 512, 2048, 2049, 4096, 8192, 9216, 32640, 131072, 1000000]


def test_decode_attention_shapes_are_launchable():
    for b, nkv, hd, ctx, combine in itertools.product(BATCHES, [1, 2, 3, 4, 8, 16, 40], [64, 128], CONTEXTS, [True, False]):
        n_splits, n_waves, lean = K._decode_shape(b, nkv, hd, ctx, combine)
        what = (b, nkv, hd, ctx, combine, n_splits, n_waves, lean)
        assert 1 <= n_splits <= 64 and n_waves in (1, 2, 4, 8) and lean in (0, 1), what
        # the kernel's LDS: a wavefront's 16 rows of head size + 2 floats, and the fused variant's queries, key and value
        lds = n_waves * 16 * (hd + 2) * 4 + 18 * hd * 2
        assert lds <= 96 * 1024, what


def test_split_counts_of_the_products_leave_no_range_empty():
    widths = [64, 72, 896, 1000, 1536, 2048, 3584, 4864, 5120, 8192, 8960, 13824, 18944, 27648, 151936]
    for m, n, k in itertools.product([1, 8, 16, 17, 32, 33, 64], widths, widths):
        s = K._n_splits(m, n, k)
        steps = -(-k // 128)
        assert 1 <= s <= steps and (s - 1) * -(-steps // s) < steps, (m, n, k, s)
    for n, k in itertools.product(widths, widths):
        s = K._f32_splits(n, k)
        steps = -(-k // 64)
        assert 1 <= s <= min(steps, 12) and (s - 1) * -(-steps // s) < steps, (n, k, s)
        s, waves = K._normed_shape(n, k)
        steps = -(-k // 128)
        assert 1 <= s <= steps and (s - 1) * -(-steps // s) < steps and waves in (4, 8, 16), (n, k, s, waves)


def test_which_rows_go_to_the_library_is_monotonic_in_the_rows():
    # up to 16 rows never, beyond 64 always, and a product that goes there at some number of rows goes there at more
    widths = [64, 896, 1536, 2048, 3584, 4608, 5120, 9728, 18944, 151936]
    for n, k in itertools.product(widths, widths):
        rows = (1, 16, 17, 24, 32, 33, 48, 64, 65, 2048)
        goes = [K._library_rows(m, n, k) for m in rows]
        assert goes[:2] == [False, False] and goes[-2:] == [True, True], (n, k, goes)
        assert goes == sorted(goes), (n, k, goes)
