"""The one rule that says which kernel serves a matrix product (``csrc/host/choice.cpp``), which the native step program
and ``ops.kernels.linear`` both ask: swept over the projections of five model shapes and every row count a step may
bring, every answer must be one that the named kernel accepts. No GPU is touched."""

import pytest
import torch

from mini_engine_amd.ops import kernels as K

# hidden, heads, kv heads, head size, intermediate (Qwen3 0.6B, 1.7B, 4B, 8B, 32B: their config.json sizes)
SHAPES = {
    "0.6b": (1024, 16, 8, 128, 3072),
    "1.7b": (2048, 16, 8, 128, 6144),
    "4b": (2560, 32, 8, 128, 9728),
    "8b": (4096, 32, 8, 128, 12288),
    "32b": (5120, 64, 8, 128, 25600),
}
VOCAB = 151936
BF16, F32 = torch.bfloat16, torch.float32


def projections(shape):
    hidden, heads, kv, d, inter = SHAPES[shape]
    return [("qkv", (heads + 2 * kv) * d, hidden, False, K.ROLE_PLAIN), ("o", hidden, heads * d, False, K.ROLE_DELTA),
            ("gate_up", 2 * inter, hidden, True, K.ROLE_PLAIN), ("down", hidden, inter, False, K.ROLE_DELTA),
            ("head", VOCAB, hidden, False, K.ROLE_HEAD)]


def accepted(kernel, rows, rows_of_w, k, gated, runs, partial, out_dtype):
    """What each kernel's entry point takes (the limits its wrapper in ops/kernels.py states)."""
    if kernel == K.PRODUCT_SMALL:
        return rows <= K.SMALL_MAX_ROWS and k % 8 == 0 and runs == 1
    if kernel == K.PRODUCT_STREAM:
        plain_f32 = not gated and (partial or out_dtype is F32)
        return (rows <= K.STREAM_MAX_ROWS and k % 8 == 0 and rows_of_w * k * 2 < 2**31 and (runs == 1 or plain_f32)
                and 1 <= runs <= 16 and (runs == 1 or rows <= 64))
    if kernel == K.PRODUCT_TILED:
        return k % 64 == 0 and runs == 1
    return kernel == K.PRODUCT_LIBRARY and runs == 1


@pytest.mark.parametrize("shape", sorted(SHAPES))
@pytest.mark.parametrize("units", [256, 304, 104])
def test_every_choice_is_one_its_kernel_accepts(shape, units):
    kernels_seen = set()
    for name, rows_of_w, k, gated, role in projections(shape):
        out_dtype = F32 if role == K.ROLE_HEAD else BF16
        for rows in list(range(1, 301)) + [512, 2048, 8192]:
            kernel, runs, partial, gate_after = K.product_choice(BF16, role, rows, rows_of_w, k, gated, out_dtype, units)
            assert accepted(kernel, rows, rows_of_w, k, gated and not gate_after, runs, partial, out_dtype), (name, rows, kernel, runs)
            assert partial == (role == K.ROLE_DELTA) and (not gate_after or gated)
            if gate_after:  # a gate behind the product needs the whole product first
                assert kernel == K.PRODUCT_LIBRARY
            kernels_seen.add(kernel)
            # the float32 path knows one product
            assert K.product_choice(F32, role, rows, rows_of_w, k, gated, F32, units) == (K.PRODUCT_F32, 1, False, gated)
    assert K.PRODUCT_STREAM in kernels_seen and K.PRODUCT_LIBRARY in kernels_seen


def test_sizes_no_kernel_of_the_package_takes_go_to_the_library():
    for rows in (1, 16, 64, 300):
        assert K.product_choice(BF16, K.ROLE_PLAIN, rows, 100, 36, False, BF16, 256)[0] == K.PRODUCT_LIBRARY  # k % 8
        assert K.product_choice(BF16, K.ROLE_PLAIN, rows, 96, 64, False, BF16, 256, aligned=False)[0] == K.PRODUCT_LIBRARY
        kernel, runs, partial, _ = K.product_choice(BF16, K.ROLE_DELTA, rows, 100, 36, False, BF16, 256)
        assert (kernel, runs, partial) == (K.PRODUCT_LIBRARY, 1, True)
    for rows in (1, 8, 32, 64):  # 2 GiB of weight: beyond what the weight-streaming kernel addresses
        for role in (K.ROLE_PLAIN, K.ROLE_DELTA, K.ROLE_HEAD):
            assert K.product_choice(BF16, role, rows, 2**20, 1024, False, BF16, 256)[0] != K.PRODUCT_STREAM


def test_the_measured_rules_at_their_shapes():
    """What the measurements beside the rules decided, at the sizes they were taken at."""
    pick = lambda role, rows, rows_of_w, k, gated=False, out=BF16: K.product_choice(BF16, role, rows, rows_of_w, k, gated, out, 256)[:2]
    assert pick(K.ROLE_PLAIN, 8, 4096, 1024) == (K.PRODUCT_SMALL, 1) and pick(K.ROLE_PLAIN, 32, 4096, 1024) == (K.PRODUCT_STREAM, 1)
    assert pick(K.ROLE_PLAIN, 8, 6144, 4096) == (K.PRODUCT_STREAM, 1) and pick(K.ROLE_PLAIN, 48, 6144, 4096) == (K.PRODUCT_LIBRARY, 1)
    assert pick(K.ROLE_DELTA, 8, 1024, 3072) == (K.PRODUCT_STREAM, 6) and pick(K.ROLE_DELTA, 65, 1024, 3072) == (K.PRODUCT_LIBRARY, 1)
    assert pick(K.ROLE_PLAIN, 128, 6144, 1024, True) == (K.PRODUCT_STREAM, 1) and pick(K.ROLE_PLAIN, 2048, 6144, 1024, True) == (K.PRODUCT_TILED, 1)
    assert pick(K.ROLE_PLAIN, 2048, 24576, 4096, True) == (K.PRODUCT_LIBRARY, 1)
    assert pick(K.ROLE_HEAD, 1, VOCAB, 1024, out=F32) == (K.PRODUCT_SMALL, 1) and pick(K.ROLE_HEAD, 8, VOCAB, 1024, out=F32) == (K.PRODUCT_STREAM, 1)
    assert pick(K.ROLE_HEAD, 64, VOCAB, 1024, out=F32) == (K.PRODUCT_LIBRARY, 1)
    fusion = lambda rows, rows_of_w, k, pending: K.lib().me_norm_fusion_choice(1, rows, rows_of_w, k, pending, 256, 1)
    assert fusion(1, 4096, 1024, 2) == K.NORM_IN_STREAM and fusion(8, 4096, 1024, 1) == K.NORM_IN_SMALL
    assert fusion(8, 4096, 1024, 2) == K.NORM_ALONE and fusion(8, 6144, 4096, 1) == K.NORM_ALONE and fusion(17, 4096, 1024, 0) == K.NORM_ALONE


@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_a_delta_is_added_into_the_stream_only_by_the_library(shape):
    """Up to 64 rows the step program sums partial sums of runs of k; beyond, the library adds its one product into
    the stream in its epilogue, and a shape the library is the fallback for stays one partial sum or the library's."""
    for name, rows_of_w, k, gated, role in projections(shape):
        if role != K.ROLE_DELTA:
            continue
        for rows in list(range(1, 301)) + [2048, 8192]:
            kernel, runs, partial, adds = K.delta_choice(rows, rows_of_w, k, 256)
            assert partial != adds, (name, rows)
            assert adds == (kernel == K.PRODUCT_LIBRARY), (name, rows, kernel)
            plain = K.product_choice(BF16, K.ROLE_DELTA, rows, rows_of_w, k, False, BF16, 256)
            assert (kernel, runs) == plain[:2]  # the same kernel either way: only where the sum happens differs
            if rows > 64:
                assert adds


@pytest.mark.parametrize("shape", sorted(SHAPES))
def test_a_norm_is_left_to_the_product_behind_it_only_where_that_product_scales_its_rows(shape):
    """A delta adds itself to the stream and leaves the norm behind it half done for a few rows of a small weight,
    and only in front of a product whose kernel multiplies its rows by the rest of the norm."""
    proj = {name: (rows_of_w, k, gated) for name, rows_of_w, k, gated, _ in projections(shape)}
    seen = set()
    for delta, behind in (("o", "gate_up"), ("down", "qkv")):
        n, k, _ = proj[delta]
        next_rows, hidden, gated = proj[behind]
        assert hidden == n
        for rows in list(range(1, 301)) + [2048]:
            carried = K.carried_norm_choice(BF16, rows, n, k, next_rows, gated, 256)
            seen.add(carried)
            if carried:
                assert 3 <= rows <= 16 and n * k * 2 < 16 << 20
                kernel, _, partial, gate_after = K.product_choice(BF16, K.ROLE_PLAIN, rows, next_rows, n, gated, BF16, 256)
                assert kernel in (K.PRODUCT_SMALL, K.PRODUCT_STREAM) and not gate_after and not partial
            assert not K.carried_norm_choice(F32, rows, n, k, next_rows, gated, 256)
            assert not K.carried_norm_choice(BF16, rows, n, k, next_rows, gated, 256, aligned=False)
    assert (True in seen) == (shape in ("0.6b", "1.7b"))


def test_the_tiny_models_of_the_gpu_tests_leave_their_norms_to_the_products_behind():
    """The GPU tests replay steps of three to sixteen tokens on these models: the carried norm is what they run there
    (all but E, whose widths no kernel of this kind takes)."""
    from conftest import tiny_configs

    for name, cfg in tiny_configs().items():
        hidden, inter, width = cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads * cfg.head_dim
        qkv_rows = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
        for rows in (3, 8, 16):
            assert K.carried_norm_choice(BF16, rows, hidden, width, 2 * inter, True, 256) == (name != "E"), name
            assert K.carried_norm_choice(BF16, rows, hidden, inter, qkv_rows, False, 256) == (name != "E"), name


def test_the_output_projection_adds_up_the_splits_of_one_item_for_narrow_models_only():
    """One item a step, up to 1,024 hidden columns: the output projection behind decode attention reads the splits'
    partial results itself (the 0.6B shape and the tiny models C and D, whose head sizes its kernel takes); wider
    models, more items and float32 keep the kernel that adds the splits up."""
    from conftest import tiny_configs

    for shape, (hidden, heads, kv, d, inter) in SHAPES.items():
        for rows in (1, 2, 3, 8, 64):
            assert K.split_sum_choice(BF16, rows, hidden) == (rows == 1 and shape == "0.6b"), (shape, rows)
            assert not K.split_sum_choice(F32, rows, hidden)
            assert not K.split_sum_choice(BF16, rows, hidden, aligned=False)
    for name in ("C", "D"):
        cfg = tiny_configs()[name]
        assert K.split_sum_choice(BF16, 1, cfg.hidden_size) and not K.split_sum_choice(BF16, 2, cfg.hidden_size)
