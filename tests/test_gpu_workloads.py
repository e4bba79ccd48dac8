'''The benchmark workloads end to end through vkjax_amd.wrap against the CPU oracle, at sizes
the oracle finishes in seconds; tolerances are the north-star ones (bit-exact RNG / gather /
argmax, 1e-5 element-wise and reductions, 1e-4 dot and conv, 1e-3 ResNet logits).'''
import threading

import numpy as np
import pytest

import vkjax_amd
from vkjax_amd import kernels as K, minijax as mj, workloads as W
from tests.common import check_against_oracle, assert_tree_close, oracle_outputs

pytestmark = pytest.mark.gpu


def test_affine():
    check_against_oracle(W.affine, W.affine_inputs(), rtol=1e-4, atol=1e-6)


def test_mlp():
    (probs, labels), (probs_true, labels_true), _ = check_against_oracle(W.mlp, W.mlp_inputs(), rtol=1e-4, atol=1e-6)
    assert np.allclose(probs.sum(axis=1), 1.0, atol=1e-5)


def test_conv_block_small_and_full():
    check_against_oracle(W.conv_block, W.conv_block_inputs(batch=2, size=14, channels=16), rtol=1e-4, atol=1e-5)
    check_against_oracle(W.conv_block, W.conv_block_inputs(), rtol=1e-4, atol=1e-5)


def test_resnet50_reduced_width():
    '''The full layer graph (53 convolutions) at a quarter of the channel widths, batch 2, 64x64 images.'''
    args = W.resnet50_inputs(batch=2, size=64, num_classes=40, width_scale=0.25)
    (logits, labels), (logits_true, labels_true), _ = check_against_oracle(W.resnet50, args, rtol=1e-3, atol=1e-4)
    assert labels.dtype == np.int32


def test_resnet50_reduced_width_single_image():
    '''Batch of one (dimensions of size 1 in every activation).'''
    args = W.resnet50_inputs(batch=1, size=64, num_classes=40, width_scale=0.25)
    check_against_oracle(W.resnet50, args, rtol=1e-3, atol=1e-4)


def test_resnet50_full_width_batch2():
    '''rtol 1e-3 on the logits. With random He-normal weights the logits reach several thousand while
    individual ones pass through zero, so the absolute floor is tied to their scale: 1e-5 of the
    largest logit (fp32 rounding of sums of that size), not a fixed 1e-4.'''
    args = W.resnet50_inputs(batch=2, size=224)
    (logits_true, labels_true), _ = oracle_outputs(W.resnet50, args)
    logits, labels = vkjax_amd.wrap(W.resnet50, frontend='minijax')(*args)
    scale = float(np.abs(logits_true).max())
    assert np.allclose(logits, logits_true, rtol=1e-3, atol=1e-5 * scale), float(np.abs(logits - logits_true).max())
    assert np.array_equal(labels, labels_true)


def test_resnet50_batch64_against_its_own_batch_of_two():
    '''The benchmark configuration itself (batch 64, 224 x 224), too long for the oracle, through what does not
    depend on the batch size: an image's logits do not depend on its neighbours, so (1) the first two rows equal
    a batch-of-two evaluation of the same images (which the test above pins to the oracle) within the logits'
    tolerance (the two sizes use different tiles and k splits, so not bit for bit), (2) copies of an image placed
    elsewhere in the batch give the same bits where the same tiling computes them (the last images of the batch
    fall into the rows that the layers with few tiles compute as 32 x 32 tiles with a four-way k split: the same
    values within the tolerance of a sum taken in another order), and (3) every label is the index of its row's
    largest logit.'''
    params, x = W.resnet50_inputs(batch=64, size=224)
    x = x.copy()
    x[63], x[32], x[20] = x[0], x[1], x[0]
    logits, labels = vkjax_amd.wrap(W.resnet50, frontend='minijax')(params, x)
    logits2, labels2 = vkjax_amd.wrap(W.resnet50, frontend='minijax')(params, x[:2].copy())
    assert logits.shape == (64, 1000) and np.all(np.isfinite(logits))
    scale = float(np.abs(logits2).max())
    assert np.allclose(logits[:2], logits2, rtol=1e-3, atol=1e-5 * scale), float(np.abs(logits[:2] - logits2).max())
    assert np.array_equal(logits[20], logits[0]) and np.array_equal(logits[32], logits[1])
    assert np.allclose(logits[63], logits[0], rtol=1e-4, atol=1e-5 * scale), float(np.abs(logits[63] - logits[0]).max())
    assert np.array_equal(labels, np.argmax(logits, axis=1).astype(labels.dtype))
    assert np.array_equal(labels[:2], labels2)


def test_rng_small_and_full_bit_exact():
    check_against_oracle(lambda key: W.rng_uniform(key, (5, 7)), W.rng_inputs(), exact=True)
    y, ytrue, _ = check_against_oracle(W.rng_uniform, W.rng_inputs(), exact=True)
    assert y.shape == (4096, 4096) and y.dtype == np.float32
    assert 0.0 <= y.min() and y.max() < 1.0 and abs(y.mean() - 0.5) < 1e-3


def test_randint_bit_exact():
    '''jax.random.randint as the reference tests it (reference: tests/test_random.py:45-60: seed 0 and 50 random
    seeds, shape [1], bounds 0 and 9999), then larger draws, negative and reversed bounds, a span over 2**16 (whose
    products wrap in 32 bits, as they do in jax) and an upper bound beyond int32.'''
    r = mj.random
    fn = lambda k: r.randint(k, [1], 0, 9999)
    wrapped = vkjax_amd.wrap(fn, frontend='minijax')
    for seed in [0] + list(np.random.RandomState(3).randint(10000, size=50)):
        key = r.PRNGKey(int(seed))
        assert np.array_equal(wrapped(key), oracle_outputs(fn, [key])[0]), seed
    for shape, lo, hi in (((257, 33), -5, 17), ((1000,), 0, 2**31 - 1), ((64, 64), 0, 2**31), ((5,), 7, 7), ((5,), 9, -9), ((4096,), 0, 100000)):
        print(f'randint {shape} [{lo}, {hi})', flush=True)
        y, _, _ = check_against_oracle(lambda k: r.randint(k, shape, lo, hi), [r.PRNGKey(11)], exact=True)
        assert y.dtype == np.int32 and (y >= lo).all() and (y.astype(np.int64) < max(hi, lo + 1)).all()


def test_random_stream_fusion_variants_bit_exact():
    '''The fused counter + block function + concatenate + chain launch against the oracle's
    one-primitive-at-a-time evaluation: lengths that are and are not multiples of 8 (16-byte and
    4-byte stores), odd lengths (the legacy layout pads the counters and trims the result, which
    keeps the chain a launch of its own), a range given at run time (scalar operands read from
    device memory), raw bits, and a split feeding two draws.'''
    from vkjax_amd.minijax import random as mrandom
    key = W.rng_inputs()

    def ranged(key, lo, hi):
        u = mrandom.uniform(key, (64, 48))
        return u * (hi - lo) + lo

    def two_draws(key):
        k1, k2 = mrandom.split(key)
        return mrandom.uniform(k1, (24,)), mrandom.random_bits(k2, (6, 4))

    cases = [(lambda key: mrandom.uniform(key, (40,)), key), (lambda key: mrandom.uniform(key, (6,)), key),
             (lambda key: mrandom.uniform(key, (7, 3)), key), (lambda key: mrandom.uniform(key, (1,)), key),
             (lambda key: mrandom.random_bits(key, (128,)), key), (lambda key: mrandom.uniform(key, (16, 8), minval=-3.0, maxval=5.0), key),
             (ranged, list(key) + [np.float32(-2.0), np.float32(7.5)]), (two_draws, key)]
    for i, (f, args) in enumerate(cases):
        _, _, fn = check_against_oracle(f, args, exact=True)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        if i not in (2, 3):                       #odd lengths keep the unfused launches
            assert any(k.startswith('threefry2x32_stream') for k in kernels), kernels
            assert not any(k.startswith(('iota', 'concat')) for k in kernels), kernels


def test_gather_scatter_small_exact_and_full():
    #integer-valued updates make the atomic sums exact whatever their order
    rng = np.random.default_rng(0)
    table   = rng.random((97, 12), dtype=np.float32)
    idx     = rng.integers(-97, 97, size=(33, 5)).astype(np.int32)
    updates = rng.integers(-5, 6, size=(33, 5, 12)).astype(np.float32)
    check_against_oracle(W.gather_scatter, [table, idx, updates], exact=True)
    table, idx, updates = W.gather_scatter_inputs()
    f = vkjax_amd.wrap(W.gather_scatter, frontend='minijax')
    rows, acc = f(table, idx, updates)
    assert np.array_equal(rows, table[idx])
    expected = np.zeros(table.shape, np.float64)
    np.add.at(expected, idx.reshape(-1), updates.reshape(-1, table.shape[1]).astype(np.float64))
    assert np.allclose(acc, expected, rtol=1e-5, atol=1e-6)


def test_scatter_add_rows_sorted_and_atomic_paths():
    '''Row scatter-add through both implementations (buckets from a counting sort of the indices; HBM atomics):
    integer-valued updates make every sum exact. Cases cover rows that receive no update, rows that receive more
    than 16 and more than 64, indices outside the table (dropped), row lengths that are not a multiple of 4 or
    longer than one pass of a wave, integer data, operands that are not zero, more than 256 x 1024 table rows
    (bucket starts in segments of several tiles), a constant table filled with one value (not read at all), and
    evaluating twice (the counters go back to zero). The sorted path runs with the table of fixed-capacity buckets
    as the host would size it, without it (every update goes through the overflow table), and with 4 and 64 slots per
    row: rows within their slots, rows beyond them and both in one program.'''
    from vkjax_amd import ops
    rng = np.random.default_rng(7)

    def scatter(table, idx, updates):
        return mj.numpy.index_add(table, idx, updates)

    def scatter_into_constant(fill):
        def f(idx, updates):
            return mj.numpy.index_add(mj.numpy.full((300, 64), fill, np.float32), idx, updates)
        return f

    for path, threshold, cap in (('sum', 0, None), ('sum', 0, 0), ('sum', 0, 4), ('sum', 0, 64), ('atomic', 1 << 60, None)):
        print(f'case: row scatter-add, {path} path, {cap} slots per row', flush=True)
        with K.overrides(scatter_sort_threshold=threshold, scatter_bucket_cap=cap):
            cases = [(50, 256, 400, np.float32), (9, 10, 37, np.float32), (300, 64, 200, np.int32), (4, 20, 500, np.float32),
                     (3000, 16, 9000, np.float32), (70, 520, 300, np.float32), (5, 8, 20000, np.int32), (1029, 4, 30000, np.float32),
                     (300000, 4, 5000, np.float32), (1025, 4, 3000, np.int32), (1024, 4, 3000, np.int32), (1023, 4, 3000, np.int32)]
            for rows, cols, n, dtype in cases:
                table   = rng.integers(-9, 9, size=(rows, cols)).astype(dtype)
                idx     = rng.integers(0, rows, size=(n,)).astype(np.int32)
                idx[: n // 3] = idx[0]                                 #one crowded row
                idx[n // 3: n // 3 + 20] = (idx[0] + 1) % rows         #and one with 20 or so
                updates = rng.integers(-5, 6, size=(n, cols)).astype(dtype)
                _, _, fn = check_against_oracle(scatter, [table, idx, updates], exact=True)
                kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
                assert any(k.startswith('scatter_rows_sum') for k in kernels) == (path == 'sum'), kernels
                #again, other values: nothing may be left over from the first evaluation
                updates2 = rng.integers(-5, 6, size=(n, cols)).astype(dtype)
                idx2     = rng.permutation(idx)
                expected = table.copy()
                np.add.at(expected, idx2, updates2)
                assert np.array_equal(fn(table, idx2, updates2), expected), (path, rows, cols, n)
                interp = list(fn._jaxpr_interpreters.values())[0]
                for key, b in interp.bufferpool.buffers.items():
                    if isinstance(key, tuple) and key[:1] == ('zeroed',):
                        words = b.numpy().reshape(-1)
                        #(the word behind the counters is the cursor that the bucketing launch resets itself)
                        assert not (words[:-1] if key[2] == 'counters' else words).any(), 'counters and overflow table are zero after an evaluation'
                if path == 'sum' and cap is not None:
                    rank_launch = [l for l in interp.launches if l.kernel == 'scatter_rows_rank'][0]
                    assert np.frombuffer(rank_launch.params, np.uint32)[7] == cap
                    assert rank_launch.buffers[1][0].size == (rows * cap if cap else n)
            #indices beyond the table (jnp's normalisation only wraps negative ones)
            table   = np.zeros((16, 8), np.float32)
            idx     = np.array([3, 99, 16, 15, -1, 3], np.int32)
            updates = rng.integers(-5, 6, size=(6, 8)).astype(np.float32)
            check_against_oracle(scatter, [table, idx, updates], exact=True)
            #a constant table of one value
            for fill in (0.0, -3.0):
                idx     = rng.integers(0, 300, size=(700,)).astype(np.int32)
                updates = rng.integers(-5, 6, size=(700, 64)).astype(np.float32)
                _, _, fn = check_against_oracle(scatter_into_constant(fill), [idx, updates], exact=True)
                if path == 'sum':
                    launch = [l for l in list(fn._jaxpr_interpreters.values())[0].launches if l.kernel.startswith('scatter_rows_sum')][0]
                    assert launch.buffers[1][0].size == 1, 'the constant table should have been replaced by its value'


def test_binding_repeated_equations_to_one_buffer_changes_no_bit():
    '''An equation that repeats an earlier one is bound to that one's buffer: programs in which that happens (the
    index normalisation of a gather followed by a scatter-add, repeated views and element-wise steps) give the same
    bits with the pass switched off, fused and unfused.'''
    rng = np.random.default_rng(23)
    def views_and_chains(x, y):
        a = (x + 1.0) * (x + 1.0)
        b = x.reshape(-1)[::2] + x.reshape(-1)[::2]
        c = mj.numpy.exp(x.T) - mj.numpy.exp(x.T) * y.T
        return a + y, b, c, (x + 1.0).sum(axis=0)
    #(integer-valued updates: the atomic additions of a small scatter-add come in any order)
    idx = rng.integers(-40, 40, size=(64, 3)).astype(np.int32)
    table, idx2, updates = W.gather_scatter_inputs(rows=512, cols=256, n0=256, n1=8)
    programs = [(W.gather_scatter, [rng.random((40, 24), dtype=np.float32), idx, rng.integers(-9, 10, size=(64, 3, 24)).astype(np.float32)]),
                (W.gather_scatter, [table, idx2, np.round(updates * 16)]),
                (views_and_chains, [rng.random((18, 32), dtype=np.float32), rng.random((18, 32), dtype=np.float32)])]
    for f, args in programs:
        for fuse in (True, False):
            with K.overrides(reuse_equal_equations=True):
                bound = vkjax_amd.wrap(f, frontend='minijax', fuse=fuse)
                y = bound(*args)
            with K.overrides(reuse_equal_equations=False):
                plain = vkjax_amd.wrap(f, frontend='minijax', fuse=fuse)
                ytrue = plain(*args)
            count = lambda fn: len(list(fn._jaxpr_interpreters.values())[0].launches)
            #(fused, the index normalisations of a gather and a scatter-add vanish into their kernels either way)
            assert count(bound) < count(plain) or (fuse and f is W.gather_scatter and count(bound) == count(plain)), (f.__name__, fuse, count(bound), count(plain))
            assert_tree_close(y, ytrue, exact=True, what=f'{f.__name__} fuse={fuse}')


def test_sorted_scatter_add_adds_in_update_order():
    '''Rows that receive up to 4096 updates are summed as operand + u(i0) + u(i1) + ... in ascending update number,
    whatever order the threads ran in: with random float data the result equals numpy's sequential float32
    accumulation (np.add.at) bit for bit, and a second evaluation gives the same bits. Buckets of 1, 64, 65, 200,
    1000 and 4096 entries, and one of 6000, which is summed in blocks whose membership may vary: that row is
    compared within the tolerance of a float32 sum.'''
    rng = np.random.default_rng(31)
    rows, cols = 600, 64
    sizes = {3: 1, 10: 64, 11: 65, 20: 200, 21: 1000, 30: 4096, 40: 6000}
    idx = np.concatenate([np.full(n, r, np.int32) for r, n in sizes.items()] + [rng.integers(100, rows, size=3000).astype(np.int32)])
    rng.shuffle(idx)
    table   = rng.standard_normal((rows, cols)).astype(np.float32)
    updates = rng.standard_normal((idx.size, cols)).astype(np.float32)
    expected = table.copy()
    np.add.at(expected, idx, updates)                          #sequential, in update order, in float32
    with K.overrides(scatter_sort_threshold=0):
        fn = vkjax_amd.wrap(lambda t, i, u: mj.numpy.index_add(t, i, u), frontend='minijax')
        first  = fn(table, idx, updates)
        second = fn(table, idx, updates)
    kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
    assert any(k.startswith('scatter_rows_sum') for k in kernels), kernels
    crowded = 40
    others = np.arange(rows) != crowded
    assert np.array_equal(first[others], expected[others])
    assert np.array_equal(first[others], second[others])
    assert np.allclose(first[crowded], expected[crowded], rtol=1e-4, atol=1e-3)
    #integer data: exact everywhere, the crowded row included
    itable, iupdates = np.round(table * 4).astype(np.int32), np.round(updates * 4).astype(np.int32)
    iexpected = itable.copy()
    np.add.at(iexpected, idx, iupdates)
    with K.overrides(scatter_sort_threshold=0):
        assert np.array_equal(vkjax_amd.wrap(lambda t, i, u: mj.numpy.index_add(t, i, u), frontend='minijax')(itable, idx, iupdates), iexpected)


def test_index_normalisation_is_done_by_the_indexing_kernels():
    '''`table[i]` and `table.at[i].add(u)` with indices that count from the end: the normalisation select(i < 0, i + n, i)
    is no launch of its own where a row gather or a sorted row scatter-add reads it, also when both read the same
    indices; where something else reads the normalised indices too, or the scatter-add is an atomic one, it stays.'''
    rng = np.random.default_rng(41)
    table   = rng.integers(-9, 9, size=(500, 32)).astype(np.float32)
    idx     = rng.integers(-500, 500, size=(40, 7)).astype(np.int32)
    idx[0, :3] = [-500, -1, 499]
    updates = rng.integers(-5, 6, size=(40, 7, 32)).astype(np.float32)
    names = lambda fn: [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
    with K.overrides(scatter_sort_threshold=0):
        _, _, fn = check_against_oracle(W.gather_scatter, [table, idx, updates], exact=True)
        assert names(fn) == ['gather_rows_v4', 'scatter_rows_rank', 'scatter_rows_sum_f_v4'], names(fn)
        _, _, fn = check_against_oracle(lambda t, i: t[i], [table, idx], exact=True)
        assert names(fn) == ['gather_rows_v4']
        _, _, fn = check_against_oracle(lambda t, i, u: mj.numpy.index_add(t, i, u), [table, idx, updates], exact=True)
        assert names(fn)[0] == 'scatter_rows_rank', names(fn)
        #the normalised indices are a result as well: they have to exist
        _, _, fn = check_against_oracle(lambda t, i: (t[i], mj.lax.select(i < 0, i + 500, i)), [table, idx], exact=True)
        assert names(fn)[0].startswith('ew_chain'), names(fn)
    with K.overrides(scatter_sort_threshold=1 << 60):
        _, _, fn = check_against_oracle(W.gather_scatter, [table, idx, updates], exact=True)
        assert names(fn)[0].startswith('ew_chain') and 'scatter_add_rows' in names(fn), names(fn)
    check_against_oracle(W.gather_scatter, [table, idx, updates], exact=True, fuse=False)


def test_failed_evaluation_leaves_the_scatter_counters_zero():
    '''The sorted scatter-add counts in an array that every evaluation leaves zero again - if it runs to the end.
    After an evaluation that failed half way the interpreter writes the zeros again, so the next one is right.'''
    from vkjax_amd import hip
    rng = np.random.default_rng(17)
    table   = rng.integers(-9, 9, size=(300, 64)).astype(np.float32)
    idx     = rng.integers(0, 300, size=(2000,)).astype(np.int32)
    updates = rng.integers(-5, 6, size=(2000, 64)).astype(np.float32)
    expected = table.copy()
    np.add.at(expected, idx, updates)
    with K.overrides(scatter_sort_threshold=0):
        fn = vkjax_amd.wrap(lambda t, i, u: mj.numpy.index_add(t, i, u), frontend='minijax')
        assert np.array_equal(fn(table, idx, updates), expected)
    interp = list(fn._jaxpr_interpreters.values())[0]
    counters = [b for key, b in interp.bufferpool.buffers.items() if isinstance(key, tuple) and key[:1] == ('zeroed',)]
    assert counters
    real = interp.sequence.eval
    def stopped_half_way(*args, **kwargs):
        for b in counters:
            b.tensor.upload(np.full(b.size, 7, np.uint32))     #what the counting launch leaves when the ordering launch never ran
        raise hip.HipError('injected failure')
    interp.sequence.eval = stopped_half_way
    with pytest.raises(hip.HipError, match='injected'):
        fn(table, idx, updates)
    interp.sequence.eval = real
    for b in counters:
        assert not b.numpy().any()
    assert np.array_equal(fn(table, idx, updates), expected)


def test_fusion_does_not_change_a_single_bit():
    '''The fused program (chains merged, batch-norm / ReLU / residual in the convolution epilogue)
    performs the same fp32 operations in the same order as one launch per equation.'''
    from vkjax_amd.minijax import tree_util
    cases = [(W.mlp, W.mlp_inputs()), (W.conv_block, W.conv_block_inputs(batch=3, size=20, channels=24)),
             (W.resnet50, W.resnet50_inputs(batch=2, size=64, num_classes=40, width_scale=0.25)),
             (lambda key: W.rng_uniform(key, (33, 20)), W.rng_inputs())]
    for f, args in cases:
        fused   = vkjax_amd.wrap(f, frontend='minijax', fuse=True)
        unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)
        a, b = fused(*args), unfused(*args)
        n_fused   = len(list(fused._jaxpr_interpreters.values())[0].launches)
        n_unfused = len(list(unfused._jaxpr_interpreters.values())[0].launches)
        assert n_fused < n_unfused
        assert_tree_close(a, b, exact=True, what=getattr(f, '__name__', 'f'))


def test_softmax_with_its_argmax_in_one_launch():
    '''softmax over rows followed by the arg-max of the probabilities becomes one launch; probabilities and labels
    equal the unfused program's bit for bit, with ties (first occurrence), NaN rows (the first NaN), rows of equal
    values, -inf entries, row lengths below and above one pass of a wave, and labels that are also a result when the
    probabilities are not.'''
    rng = np.random.default_rng(5)
    def probabilities_and_labels(x):
        p = mj.nn.softmax(x, axis=-1)
        return p, mj.numpy.argmax(p, axis=1)
    def labels_only(x):
        return mj.numpy.argmax(mj.nn.softmax(x, axis=-1), axis=1)
    for rows, cols in ((256, 10), (7, 1), (33, 64), (5, 200), (4, 1000)):
        x = rng.standard_normal((rows, cols)).astype(np.float32)
        x[0, :] = 0.5                                             #all equal: label 0
        if cols > 3:
            x[1, 2], x[1, cols - 1] = 9.0, 9.0                    #a tie: the first
            x[2, cols // 2] = np.nan                              #NaN probabilities in the whole row: label 0
            x[3 % rows, 0] = -np.inf
        for f in (probabilities_and_labels, labels_only):
            fused   = vkjax_amd.wrap(f, frontend='minijax', fuse=True)
            unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)
            a, b = fused(x), unfused(x)
            kernels = [l.kernel for l in list(fused._jaxpr_interpreters.values())[0].launches]
            #rows of one value have nothing to reduce: no softmax kernel is involved there
            assert cols == 1 or (len(kernels) == 1 and kernels[0].startswith('softmax_rows')), (kernels, rows, cols)
            assert_tree_close(a, b, exact=True, what=f'{f.__name__} {rows}x{cols}')
            labels = a[1] if isinstance(a, tuple) else a
            assert labels[0] == 0 and (cols <= 3 or labels[1] == 2)


def test_products_with_few_output_features():
    '''dense_rows_n16: one wave per row on the vector ALUs for products with at most 16 output features. Every width
    from 1 to 16, contractions of one vector, several passes and a last pass that is not full, one row and row counts
    that do not fill a workgroup; bias, bias + ReLU, scale and shift, nothing; integer-valued data, so every result is
    exact against the oracle. Followed by softmax (and the arg-max of the probabilities) the whole layer is ONE
    launch whose probabilities and labels equal the unfused program's bit for bit: ties, NaN and infinite logits, a
    single class. 17 features go to the matrix-core kernels.'''
    rng = np.random.default_rng(12)
    ints = lambda lo, hi, *shape: rng.integers(lo, hi, size=shape).astype(np.float32)
    def plain(x, w): return mj.numpy.dot(x, w)
    def bias(x, w, b): return mj.numpy.dot(x, w) + b
    def bias_relu(x, w, b): return mj.nn.relu(mj.numpy.dot(x, w) + b)
    def scale_shift(x, w, m, s, b): return (mj.numpy.dot(x, w) - m) * s + b
    shapes = [(256, 512, 10), (1, 4, 1), (3, 8, 2), (5, 252, 3), (4, 256, 4), (7, 260, 5), (33, 516, 6), (2, 784, 7), (65, 1028, 8),
              (9, 64, 9), (130, 300, 11), (6, 1024, 12), (17, 2052, 13), (40, 128, 14), (3, 388, 15), (100, 768, 16)]
    for rows, k, n in shapes:
        x, w = ints(-4, 5, rows, k), ints(-3, 4, k, n)
        for f, extra in ((plain, []), (bias, [ints(-9, 9, n)]), (bias_relu, [ints(-9, 9, n)]),
                         (scale_shift, [ints(-5, 5, n), ints(1, 4, n), ints(-9, 9, n)])):
            _, _, fn = check_against_oracle(f, [x, w] + extra, exact=True)
            kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
            #(with one output feature a per-feature vector is a single value, which the general epilogue handles)
            assert kernels == ['dense_rows_n16'] or (n == 1 and f is not plain), (kernels, f.__name__, rows, k, n)
    _, _, fn = check_against_oracle(plain, [ints(-4, 5, 40, 256), ints(-3, 4, 256, 17)], exact=True)
    assert [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches] != ['dense_rows_n16']

    def head(x, w, b):
        p = mj.nn.softmax(mj.numpy.dot(x, w) + b, axis=-1)
        return p, mj.numpy.argmax(p, axis=1)
    def head_probabilities(x, w, b):
        return mj.nn.softmax(mj.numpy.dot(x, w) + b, axis=-1)
    def head_relu_labels(x, w, b):
        return mj.numpy.argmax(mj.nn.softmax(mj.nn.relu(mj.numpy.dot(x, w) + b), axis=-1), axis=1)
    for rows, k, classes in [(256, 512, 10), (7, 256, 12)] + [(9, 64, c) for c in range(1, 17)] + [(40, 256, 17)]:
        x = rng.standard_normal((rows, k)).astype(np.float32)
        w = (rng.standard_normal((k, classes)) / np.sqrt(k)).astype(np.float32)
        b = rng.standard_normal(classes).astype(np.float32)
        x[0, :] = 0.0                                             #logits = bias
        if classes > 1:
            w[:, 1] = w[:, 0]; b[1] = b[0]                        #classes 0 and 1 tie in every row
        x[2, 5] = np.nan                                          #a row of NaN logits
        x[3, 7] = np.inf                                          #logits +-inf (or NaN) in row 3
        for f in (head, head_probabilities, head_relu_labels):
            fused   = vkjax_amd.wrap(f, frontend='minijax', fuse=True)
            unfused = vkjax_amd.wrap(f, frontend='minijax', fuse=False)
            a, c = fused(x, w, b), unfused(x, w, b)
            kernels = [l.kernel for l in list(fused._jaxpr_interpreters.values())[0].launches]
            if 1 < classes <= 16:
                assert kernels == ['dense_rows_n16'], (kernels, rows, k, classes)
            elif classes > 16:
                assert len(kernels) == 2 and kernels[1].startswith('softmax_rows'), kernels
            assert_tree_close(a, c, exact=True, what=f'{f.__name__} {rows}x{k}x{classes}')
    #against the oracle
    check_against_oracle(head, [rng.standard_normal((256, 512)).astype(np.float32),
                                (rng.standard_normal((512, 10)) / 23).astype(np.float32), rng.standard_normal(10).astype(np.float32)],
                         rtol=1e-4, atol=1e-6)


def test_affine_chains_in_straight_line_code():
    '''ew_affine_v4 evaluates ((first + s1 + s2 + s3) - vsub) * vmul + vadd + full, max(., floor) without the opcode
    interpreter. Every subset of those parts, on 2-D, 4-D and (without vectors) 1-D arrays, gives the bits of the
    general chain kernel, NaN and infinite values included, and agrees with the oracle.'''
    import itertools
    from vkjax_amd import kernels as K
    rng = np.random.default_rng(21)
    r = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    for shape in ((37, 24), (2, 5, 7, 64), (4100,)):
        c = shape[-1]
        first, s1, s2, s3, full = (r(*shape) for _ in range(5))
        first.reshape(-1)[3] = np.nan; first.reshape(-1)[5] = np.inf; full.reshape(-1)[9] = -np.inf
        vsub, vmul, vadd = r(c), r(c), r(c)
        for nsum, parts in itertools.product(range(4), itertools.product((0, 1), repeat=5)):
            if len(shape) == 1 and any(parts[:3]):
                continue
            if nsum == 0 and not any(parts):
                continue
            def f(first, s1, s2, s3, vsub, vmul, vadd, full):
                v = first
                for s in (s1, s2, s3)[:nsum]:
                    v = v + s
                if parts[0]: v = v - vsub
                if parts[1]: v = v * vmul
                if parts[2]: v = v + vadd
                if parts[3]: v = v + full
                if parts[4]: v = mj.nn.relu(v)
                return v
            args = [first, s1, s2, s3, vsub, vmul, vadd, full]
            results = []
            for forced in (True, False):
                with K.overrides(ew_affine=forced):
                    fn = vkjax_amd.wrap(f, frontend='minijax')
                    results.append(fn(*args))
                    kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
                #(nine operands are two launches: a chain holds eight)
                assert all((k == 'ew_affine_v4') == forced for k in kernels) and len(kernels) <= 2, (kernels, forced, shape, nsum, parts)
            assert_tree_close(results[0], results[1], exact=True, what=f'{shape} {nsum} {parts}')
        check_against_oracle(lambda a, b, m, s, t, q: mj.nn.relu((a + b - m) * s + t + q), [first, s1, vsub, vmul, vadd, full][:6] if len(shape) > 1
                             else [first, s1, np.float32(0.5), np.float32(2.0), np.float32(-1.0), full], rtol=1e-5, atol=1e-6)
    #arrays of more than 4 M elements: the variant that skips absent operands, same bits as the general kernel
    big, res, m, k, t = r(1 << 16, 72), r(1 << 16, 72), r(72), r(72), r(72)
    big[5, 7] = np.nan
    for f, args in ((lambda x, m, k, t: mj.nn.relu((x - m) * k + t), [big, m, k, t]),
                    (lambda x, y, m, k, t: mj.nn.relu((x - m) * k + t + y), [big, res, m, k, t]),
                    (lambda x, y, z, w, t: x + y + z + w + t, [big, res, big[::-1].copy(), res[::-1].copy(), t])):
        results = []
        for forced in (None, False):
            with K.overrides(ew_affine=forced):
                fn = vkjax_amd.wrap(f, frontend='minijax')
                results.append(fn(*args))
                kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
            assert kernels == (['ew_affine_big_v4'] if forced is None else [kernels[0]]) and (forced is None or kernels[0].startswith('ew_chain')), kernels
        assert_tree_close(results[0], results[1], exact=True, what='large affine chain')
    #by itself: chains of more than four operands on arrays that are not large
    x, m, k, t = r(64, 7, 7, 64), r(64), r(64), r(64)
    _, _, fn = check_against_oracle(lambda x, m, k, t: mj.nn.relu((x - m) * k + t), [x, m, k, t], rtol=1e-5, atol=1e-6)
    assert [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches] == ['ew_affine_v4']
    _, _, fn = check_against_oracle(lambda x, m: mj.nn.relu(x - m), [x, m], rtol=1e-6)
    assert [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches] == ['ew_chain_v4_s4']


def test_transposes_of_several_inputs_share_a_launch():
    '''Copies that swap the two fastest dimensions of program inputs (a network's kernels, transposed for its backward
    pass) are hoisted to the front and run as one launch per kernel variant: 64 x 64 and 128 x 128 tiles, leading
    dimensions (3 x 3 kernels), extents that are no multiple of the tile, bit for bit.'''
    lax = mj.lax
    rng = np.random.default_rng(21)
    shapes = [(3, 3, 64, 128), (1, 1, 256, 512), (3, 3, 128, 256), (1, 1, 72, 200), (200, 136), (1, 1, 512, 128), (2, 3, 20, 36), (640, 384)]
    arrays = [rng.standard_normal(sh).astype(np.float32) for sh in shapes]
    def f(*xs):
        swapped = [lax.transpose(x, tuple(range(x.ndim - 2)) + (x.ndim - 1, x.ndim - 2)) for x in xs]
        return [lax.mul(t, np.float32(2.0)) for t in swapped[:2]] + swapped[2:]
    _, _, fn = check_against_oracle(f, arrays, exact=True)
    kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
    assert kernels.count('transpose_tiled_batch_v4') == 1 and kernels.count('transpose_tiled_batch_v4_t128') == 1, kernels
    assert not any(k in ('transpose_tiled_v4', 'transpose_tiled_v4_t128') for k in kernels), kernels
    check_against_oracle(f, arrays, exact=True, fuse=False)


def test_gather_fill_and_scatter_clip_modes():
    '''jax's indexing modes on the GPU against the oracle, bit for bit: FILL_OR_DROP gathers (rows of 5 and of 8
    words, a default and a given fill value, floats and integers, windows, a build-time index outside the table) and
    CLIP scatter-adds (atomic rows, the sorted kernels, windows). Integer-valued updates: every sum is exact.'''
    from vkjax_amd.minijax import core
    from vkjax_amd import ops
    lax = mj.lax
    G, S = core.GatherDimensionNumbers, core.ScatterDimensionNumbers
    rng = np.random.default_rng(12)
    rows_dn, rows_sd = G((1,), (0,), (0,)), S((1,), (0,), (0,))
    for width in (5, 8):
        table = rng.integers(-50, 50, size=(37, width)).astype(np.float32)
        idx   = rng.integers(-20, 60, size=(300, 1)).astype(np.int32)
        upd   = rng.integers(-9, 9, size=(300, width)).astype(np.float32)
        print(f'rows of {width}', flush=True)
        y, _, _ = check_against_oracle(lambda t, i: lax.gather(t, i, rows_dn, (1, width), mode='fill'), [table, idx], exact=True)
        assert np.isnan(y[(idx[:, 0] < 0) | (idx[:, 0] >= 37)]).all() and not np.isnan(y[(idx[:, 0] >= 0) & (idx[:, 0] < 37)]).any()
        check_against_oracle(lambda t, i: lax.gather(t, i, rows_dn, (1, width), mode='fill', fill_value=-1.5), [table, idx], exact=True)
        check_against_oracle(lambda t, i: lax.gather(t, i, rows_dn, (1, width), mode='FILL_OR_DROP'), [table.astype(np.int32), idx], exact=True)
        check_against_oracle(lambda t, i: lax.gather(t, i, rows_dn, (1, width), mode='clip'), [table, idx], exact=True)
        for fuse in (True, False):
            check_against_oracle(lambda t, i, u: lax.scatter_add(t, i, u, rows_sd, mode='clip'), [table, idx, upd], exact=True, fuse=fuse)
            check_against_oracle(lambda t, i, u: lax.scatter_add(t, i, u, rows_sd, mode='drop'), [table, idx, upd], exact=True, fuse=fuse)
    #a single index known when the program is built: inside it is a copy, outside the fill value
    table = rng.integers(-50, 50, size=(6, 4)).astype(np.float32)
    for row in (2, 9, -1):
        check_against_oracle(lambda t: lax.gather(t, np.array([[row]], np.int32), rows_dn, (1, 4), mode='fill'), [table], exact=True)
    #windows of 2 x 3 in a 7 x 5 table
    table  = rng.integers(-50, 50, size=(7, 5)).astype(np.float32)
    starts = rng.integers(-3, 8, size=(40, 2)).astype(np.int32)
    win    = rng.integers(-9, 9, size=(40, 2, 3)).astype(np.float32)
    check_against_oracle(lambda t, i: lax.gather(t, i, G((1, 2), (), (0, 1)), (2, 3), mode='fill'), [table, starts], exact=True)
    check_against_oracle(lambda t, i, u: lax.scatter_add(t, i, u, S((1, 2), (), (0, 1)), mode='clip'), [table, starts, win], exact=True)
    #the sorted (atomic-free) kernels
    table = rng.integers(-50, 50, size=(500, 64)).astype(np.float32)
    idx   = rng.integers(-100, 600, size=(K.CHOICES.scatter_sort_threshold // 64 + 7, 1)).astype(np.int32)
    upd   = rng.integers(-9, 9, size=(idx.shape[0], 64)).astype(np.float32)
    for mode in ('clip', None):
        _, _, fn = check_against_oracle(lambda t, i, u: lax.scatter_add(t, i, u, rows_sd, mode=mode), [table, idx, upd], exact=True)
        kernels = [l.kernel for l in list(fn._jaxpr_interpreters.values())[0].launches]
        assert 'scatter_rows_rank' in kernels, kernels


def test_indices_that_count_from_the_end():
    '''`x[i]` and `x.at[i].add(u)` with negative entries in i: tracing normalises the index as select(i < 0, i + n, i),
    which runs as one launch (opcode WRAP_I) whose result both the gather and the scatter-add read. Bit-exact against
    the oracle; the normalised index is also correct as a result of its own.'''
    rng = np.random.default_rng(31)
    table = rng.integers(-9, 10, size=(50, 12)).astype(np.float32)
    idx = rng.integers(-50, 50, size=(7, 9)).astype(np.int32)
    updates = rng.integers(-3, 4, size=(7, 9, 12)).astype(np.float32)
    def f(t, i, u):
        return t[i], mj.numpy.index_add(t, i, u)
    _, _, fn = check_against_oracle(f, [table, idx, updates], exact=True)
    ops_ = list(fn._jaxpr_interpreters.values())[0].all_ops
    labels = [repr(op.equation) for op in ops_]
    assert sum('add ; lt ; select' in l for l in labels) == 1, labels
    def normalised(i):
        return mj.lax.select(i < 0, i + 50, i)
    check_against_oracle(normalised, [idx], exact=True)
    check_against_oracle(lambda i: mj.lax.select(i < 0, i + 50, i) * 2, [np.array([-50, -1, 0, 49, -2147483648, 2147483647], np.int32)], exact=True)


def test_return_all_and_profiling():
    '''The debugging surface of the reference: run(..., return_all=True) returns every variable
    (reference: vkjax/kompute_jaxpr_interpreter.py:85-89) and profiling=True returns per-op timings
    labelled data2device / equations / data2host (reference: :91-95).'''
    from vkjax_amd.jaxpr_interpreter import JaxprInterpreter
    from oracle.eval_jaxpr import eval_closed_jaxpr
    args   = W.affine_inputs()
    closed = mj.make_jaxpr(W.affine)(*args)
    interp = JaxprInterpreter(closed, reuse_buffers=False, fuse=False)
    outs, env = interp.run(*args, return_all=True)
    _, env_true = eval_closed_jaxpr(closed, *args, return_env=True)
    for var, val in env_true.items():
        assert np.allclose(env[var], val, rtol=1e-4, atol=1e-6), var
    f = vkjax_amd.wrap(W.affine, profiling=True, frontend='minijax', fuse=False)
    y, info = f(*args)
    assert [label for label, _ in info][0] == 'data2device' and info[-1][0] == 'data2host'
    assert len(info) == 2 + 2 and all(dt >= 0 for _, dt in info)


def test_function_semantics_on_device():
    '''reference: tests/test_function.py:13-16,48-60'''
    def func0(x):
        return x + 1
    vk_func = vkjax_amd.Function(func0, frontend='minijax')
    assert vk_func(65) == 66
    assert vk_func(-5) == -4
    x  = np.arange(128).astype('uint32')
    y0 = vk_func(x)
    y1 = vk_func(x.astype('float32'))
    assert np.allclose(y0, y1) and y0.dtype == np.uint32 and y1.dtype == np.float32
    assert len(vk_func._jaxpr_interpreters) == 3
    with pytest.raises(TypeError):
        list(vk_func._jaxpr_interpreters.values())[0].run(1, 2)


def test_graph_replay_matches_individual_launches():
    '''The launches of a sequence issued as one captured HIP graph: several replays, with other work
    and synchronisations of the same program in between, each compared bit for bit with the result
    of the individually launched sequence; new inputs are picked up by every replay.'''
    rng = np.random.default_rng(11)
    for f, make in ((W.mlp, W.mlp_inputs), (W.conv_block, lambda: W.conv_block_inputs(batch=3, size=20, channels=24)),
                    (lambda key: W.rng_uniform(key, (64, 48)), W.rng_inputs)):
        plain = vkjax_amd.wrap(f, frontend='minijax')
        graph = vkjax_amd.wrap(f, frontend='minijax', graph=True)
        for rep in range(4):
            args = make()
            if rep:                                   #different data every time
                args = [a + np.asarray(rep, dtype=a.dtype) if isinstance(a, np.ndarray) and a.dtype == np.float32 else a for a in args]
            expected = plain(*args)
            got = graph(*args)
            assert_tree_close(got, expected, exact=True, what=f'graph replay {rep}')
            plain(*make())                            #unrelated eager work between graph launches
        interp = list(graph._jaxpr_interpreters.values())[0]
        assert interp.graph


def test_resident_arguments_are_uploaded_once():
    '''resident_argnums: a weight leaf is uploaded when the object passed for it changes, and only
    then; other arguments are copied on every call as in the reference.'''
    params, x = W.mlp_inputs()
    plain    = vkjax_amd.wrap(W.mlp, frontend='minijax')
    resident = vkjax_amd.wrap(W.mlp, frontend='minijax', resident_argnums=(0,))
    assert_tree_close(resident(params, x), plain(params, x), exact=True, what='first call')
    x2 = x[::-1].copy()
    assert_tree_close(resident(params, x2), plain(params, x2), exact=True, what='new activations, same weights')
    #a replaced leaf is picked up, the untouched ones stay where they are
    from vkjax_amd.minijax import tree_util
    leaves, structure = tree_util.tree_flatten(params)
    leaves2 = list(leaves)
    leaves2[0] = leaves[0] * np.float32(0.5)
    params2 = tree_util.tree_unflatten(structure, leaves2)
    assert_tree_close(resident(params2, x2), plain(params2, x2), exact=True, what='one weight replaced')
    interp = list(resident._jaxpr_interpreters.values())[0]
    assert len(interp._resident_leaves) == len(leaves)


def test_read_only_leaves_stay_in_hbm_without_being_asked():
    '''Plain `wrap(f)(params, x)`: leaves that cannot change under the caller's feet (numpy arrays that are not
    writeable) are uploaded once and again only when replaced; writeable ones are copied on every call, as the
    reference does with every argument (vkjax/kompute_jaxpr_interpreter.py:72-75); a read-only view of a writeable
    array counts as writeable. With resident_argnums a writeable leaf that is changed in place where the cheap
    check looks (its first and last 64 bytes) is uploaded again.'''
    from vkjax_amd.minijax import tree_util
    params, x = W.mlp_inputs()
    plain = vkjax_amd.wrap(W.mlp, frontend='minijax', resident_argnums=())
    def frozen(a):
        a = a.copy()
        a.flags.writeable = False
        return a
    def counted(f, *args):
        interp = f._get_or_create_jaxpr_interpreter(args)[0]
        real, seen = interp.sequence.eval, []
        def spy(host, *a, **kw):
            seen.append(sum(host[s] is not None for s in interp._input_slots if s is not None))
            return real(host, *a, **kw)
        interp.sequence.eval = spy
        try:
            y = f(*args)
        finally:
            interp.sequence.eval = real
        return y, seen[0]
    n = len(tree_util.tree_leaves(params))
    f = vkjax_amd.wrap(W.mlp, frontend='minijax')
    ro = tree_util.tree_map(frozen, params)
    for k, (xx, want) in enumerate([(x, n + 1), (x[::-1].copy(), 1), (x, 1)]):
        y, uploads = counted(f, ro, xx)
        assert uploads == want, (k, uploads)
        assert_tree_close(y, plain(params, xx), exact=True, what=f'read-only weights, call {k}')
    #a replaced leaf is picked up; the others stay
    leaves, structure = tree_util.tree_flatten(ro)
    ro2 = tree_util.tree_unflatten(structure, [frozen(leaves[0] * np.float32(0.5))] + list(leaves[1:]))
    y, uploads = counted(f, ro2, x)
    assert uploads == 2
    assert_tree_close(y, plain(ro2, x), exact=True, what='one read-only weight replaced')
    #writeable weights: every call copies everything, and sees changes made in place
    g = vkjax_amd.wrap(W.mlp, frontend='minijax')
    rw = tree_util.tree_map(np.copy, params)
    for k in range(3):
        tree_util.tree_leaves(rw)[0].reshape(-1)[5] += np.float32(1.0)
        y, uploads = counted(g, rw, x)
        assert uploads == n + 1, (k, uploads)
        assert_tree_close(y, plain(tree_util.tree_map(np.copy, rw), x), exact=True, what=f'writeable weights, call {k}')
    #a read-only window into a writeable array can change: copied every call
    views = tree_util.tree_map(lambda a: a.view(), rw)
    for v in tree_util.tree_leaves(views):
        v.flags.writeable = False
    h = vkjax_amd.wrap(W.mlp, frontend='minijax')
    assert counted(h, views, x)[1] == n + 1 and counted(h, views, x)[1] == n + 1
    #resident_argnums with writeable leaves: kept, unless a change shows in the first or last 64 bytes
    r = vkjax_amd.wrap(W.mlp, frontend='minijax', resident_argnums=(0,))
    assert counted(r, rw, x)[1] == n + 1 and counted(r, rw, x)[1] == 1
    first = tree_util.tree_leaves(rw)[0]
    first.reshape(-1)[3] += np.float32(2.0)
    y, uploads = counted(r, rw, x)
    assert uploads == 2
    assert_tree_close(y, plain(tree_util.tree_map(np.copy, rw), x), exact=True, what='changed in place near the start')
    first.reshape(-1)[-1] -= np.float32(2.0)
    assert counted(r, rw, x)[1] == 2


def test_stream_matches_call_by_call():
    '''Function.stream overlaps the upload of one argument tuple with the device work on the one
    before it; its results must be those of plain calls, in order: small arguments, arguments large
    enough for the chunked staging path (>= 8 MB), resident weights with one replaced on the way,
    a change of signature in the middle, one tuple only, and none at all.'''
    rng = np.random.default_rng(5)
    def scale_shift(x, w):
        return mj.numpy.tanh(x * w + 1.0), mj.numpy.sum(x, axis=0)
    plain = vkjax_amd.wrap(scale_shift, frontend='minijax')
    fast  = vkjax_amd.wrap(scale_shift, frontend='minijax')
    small = [(rng.standard_normal((33, 17)).astype(np.float32), rng.standard_normal((17,)).astype(np.float32)) for _ in range(4)]
    large = [(rng.standard_normal((1200, 2048)).astype(np.float32), rng.standard_normal((2048,)).astype(np.float32)) for _ in range(3)]
    for name, tuples in [('small', small), ('large', large), ('mixed signatures', small[:2] + large[:2] + small[2:]),
                         ('single', small[:1]), ('empty', [])]:
        expected = [plain(*t) for t in tuples]
        got = list(fast.stream(iter(tuples)))
        assert len(got) == len(expected), name
        for k, (g, e) in enumerate(zip(got, expected)):
            assert_tree_close(g, e, exact=True, what=f'{name} [{k}]')
    #a plain call after a stream sees its own arguments, not what the stream left behind
    assert_tree_close(fast(*small[3]), plain(*small[3]), exact=True, what='call after stream')

    params, x = W.mlp_inputs()
    plain_mlp = vkjax_amd.wrap(W.mlp, frontend='minijax')
    resident  = vkjax_amd.wrap(W.mlp, frontend='minijax', resident_argnums=(0,))
    from vkjax_amd.minijax import tree_util
    leaves, structure = tree_util.tree_flatten(params)
    params2 = tree_util.tree_unflatten(structure, [leaves[0] * np.float32(0.5)] + list(leaves[1:]))
    batches = [(params, x), (params, x[::-1].copy()), (params2, x), (params2, x * np.float32(2)), (params, x)]
    expected = [plain_mlp(*t) for t in batches]
    for k, (g, e) in enumerate(zip(resident.stream(batches), expected)):
        assert_tree_close(g, e, exact=True, what=f'resident weights [{k}]')

    #abandoning a stream half way leaves the function usable
    it = fast.stream(iter(small))
    next(it)
    it.close()
    assert_tree_close(fast(*small[0]), plain(*small[0]), exact=True, what='call after an abandoned stream')

    #the same with resident weights: what the helper thread had prepared ahead must not count as uploaded ...
    it = resident.stream(iter(batches))
    next(it)
    it.close()
    for k in (3, 0, 2):
        assert_tree_close(resident(*batches[k]), expected[k], exact=True, what=f'resident call {k} after an abandoned stream')
    #... and other calls of the function while a stream is suspended do not disturb it (nor it them)
    it = resident.stream(iter(batches))
    for k in range(len(batches)):
        assert_tree_close(next(it), expected[k], exact=True, what=f'suspended stream [{k}]')
        other = (k * 2 + 1) % len(batches)
        assert_tree_close(resident(*batches[other]), expected[other], exact=True, what=f'call {other} between stream results')


def test_stream_loader_may_refill_its_batch_array():
    '''A loader that hands out ONE preallocated batch array and refills it for every tuple: the stream
    takes its tuples several evaluations ahead, so it has to have copied each batch when it took it.'''
    rng = np.random.default_rng(11)
    def scale_shift(x, w):
        return x * w + 1.0
    plain  = vkjax_amd.wrap(scale_shift, frontend='minijax')
    stream = vkjax_amd.wrap(scale_shift, frontend='minijax')
    for shape in ((33, 17), (1200, 2048)):                    #inline staging, and the chunked path (>= 8 MB)
        w      = rng.standard_normal(shape[1:]).astype(np.float32)
        values = [rng.standard_normal(shape).astype(np.float32) for _ in range(9)]
        batch  = np.empty(shape, np.float32)
        def loader():
            for v in values:
                batch[...] = v
                yield batch, w
        got = [np.array(y) for y in stream.stream(loader())]
        assert len(got) == len(values)
        for k, (g, v) in enumerate(zip(got, values)):
            assert_tree_close(g, plain(v, w), exact=True, what=f'{shape} batch {k}')


def test_launches_follow_the_uploads_of_a_network():
    '''A call that copies every argument (writeable parameter arrays: the reference's semantics) sends them in the
    order of first use, the small ones side by side in one transfer, and issues the launches while later weights are
    still on their way. The results are those of the same program replayed on inputs uploaded one by one beforehand,
    bit for bit, call after call with changed weights and images; the program contains launches that reach their
    operands through a table (batched small chains at this batch size), which the runtime has to know as well.'''
    rng = np.random.default_rng(47)
    from vkjax_amd.minijax import tree_util
    params, x = W.resnet50_inputs(batch=2, size=64, num_classes=100, width_scale=0.5)
    assert sum(a.nbytes for a in tree_util.tree_leaves(params)) > (16 << 20)          #the chunked path, several checkpoints
    fn = vkjax_amd.wrap(W.resnet50, frontend='minijax')
    reference = vkjax_amd.wrap(W.resnet50, frontend='minijax')
    reference(params, x)
    interp = list(reference._jaxpr_interpreters.values())[0]
    previous = None
    for call in range(3):
        print(f'case: every argument copied, call {call}', flush=True)
        #new values in the same arrays (in place), a few arrays replaced
        for k, leaf in enumerate(tree_util.tree_leaves(params)):
            if k % 7 == call:
                leaf *= np.float32(1.0 + 0.01 * (call + 1))
        x = rng.standard_normal(x.shape).astype(np.float32)
        got = fn(params, x)
        interp.upload_inputs(params, x)
        interp.replay(1)
        whole = interp.read_outputs()
        for g, w in zip(tree_util.tree_leaves(got), whole):
            assert np.array_equal(np.asarray(g).reshape(-1), np.asarray(w).reshape(-1)), call
        flat = np.concatenate([np.asarray(g, np.float32).reshape(-1) for g in tree_util.tree_leaves(got)])
        assert np.isfinite(flat).all() and (previous is None or not np.array_equal(flat, previous))
        previous = flat
    assert any(l.members for l in interp.launches) or any('batch' in l.kernel for l in interp.launches), [l.kernel for l in interp.launches]


def test_stream_with_several_tuples_in_flight():
    '''Function.stream(..., in_flight=n) evaluates n tuples at a time, each on a device context of its own driven by
    its own thread; the results are those of plain calls, in the order of the tuples: small and large arguments,
    a change of signature in the middle, fewer tuples than lanes, none; resident weights with one replaced on the
    way; a loader that refills one batch array; a stream abandoned half way; an error raised by the iterable.'''
    rng = np.random.default_rng(6)
    def scale_shift(x, w):
        return mj.numpy.tanh(x * w + 1.0), mj.numpy.sum(x, axis=0)
    plain = vkjax_amd.wrap(scale_shift, frontend='minijax')
    fast  = vkjax_amd.wrap(scale_shift, frontend='minijax')
    small = [(rng.standard_normal((33, 17)).astype(np.float32), rng.standard_normal((17,)).astype(np.float32)) for _ in range(7)]
    large = [(rng.standard_normal((1200, 2048)).astype(np.float32), rng.standard_normal((2048,)).astype(np.float32)) for _ in range(5)]
    for lanes in (2, 3):
        for name, tuples in [('small', small), ('large', large), ('mixed signatures', small[:3] + large[:2] + small[3:] + large[2:]),
                             ('single', small[:1]), ('empty', [])]:
            expected = [plain(*t) for t in tuples]
            got = list(fast.stream(iter(tuples), in_flight=lanes))
            assert len(got) == len(expected), (lanes, name)
            for k, (g, e) in enumerate(zip(got, expected)):
                assert_tree_close(g, e, exact=True, what=f'{lanes} lanes, {name} [{k}]')
    #the function itself is not one of the lanes: calls between results of a stream do not disturb it
    it = fast.stream(iter(small), in_flight=2)
    for k in range(len(small)):
        assert_tree_close(next(it), plain(*small[k]), exact=True, what=f'suspended stream [{k}]')
        assert_tree_close(fast(*large[k % len(large)]), plain(*large[k % len(large)]), exact=True, what=f'call between results {k}')
    assert next(it, None) is None

    params, x = W.mlp_inputs()
    plain_mlp = vkjax_amd.wrap(W.mlp, frontend='minijax')
    resident  = vkjax_amd.wrap(W.mlp, frontend='minijax', resident_argnums=(0,))
    from vkjax_amd.minijax import tree_util
    leaves, structure = tree_util.tree_flatten(params)
    params2 = tree_util.tree_unflatten(structure, [leaves[0] * np.float32(0.5)] + list(leaves[1:]))
    batches = [(params, x), (params, x[::-1].copy()), (params2, x), (params2, x * np.float32(2)), (params, x), (params2, x[::-1].copy())]
    expected = [plain_mlp(*t) for t in batches]
    for repeat in range(2):                                   #(the second time the lanes exist and hold weights already)
        for k, (g, e) in enumerate(zip(resident.stream(batches, in_flight=2), expected)):
            assert_tree_close(g, e, exact=True, what=f'resident weights [{k}], pass {repeat}')

    #one preallocated batch array, refilled for every tuple: each lane has copied its tuple before the next is asked for
    def affine(x, w):
        return x * w + 1.0
    plain_affine, streamed = vkjax_amd.wrap(affine, frontend='minijax'), vkjax_amd.wrap(affine, frontend='minijax')
    for shape in ((33, 17), (1200, 2048)):
        w      = rng.standard_normal(shape[1:]).astype(np.float32)
        values = [rng.standard_normal(shape).astype(np.float32) for _ in range(11)]
        batch  = np.empty(shape, np.float32)
        def loader():
            for v in values:
                batch[...] = v
                yield batch, w
        got = [np.array(y) for y in streamed.stream(loader(), in_flight=2)]
        assert len(got) == len(values)
        for k, (g, v) in enumerate(zip(got, values)):
            assert_tree_close(g, plain_affine(v, w), exact=True, what=f'{shape} refilled batch {k}')

    #abandoned half way: the lanes' threads end, the function and a new stream work
    it = fast.stream(iter(small), in_flight=2)
    next(it)
    it.close()
    assert_tree_close(fast(*small[0]), plain(*small[0]), exact=True, what='call after an abandoned stream')
    assert len(list(fast.stream(iter(small), in_flight=2))) == len(small)
    assert not [t for t in threading.enumerate() if t.name.startswith('vkjax-stream-lane')]

    #an error of the iterable reaches the consumer, after the results of the tuples before it or instead of them
    def failing():
        yield small[0]
        yield small[1]
        raise KeyError('no third batch')
    with pytest.raises(KeyError, match='no third batch'):
        list(fast.stream(failing(), in_flight=2))
    assert not [t for t in threading.enumerate() if t.name.startswith('vkjax-stream-lane')]


def test_first_launch_starts_while_its_argument_arrives():
    '''A convolution over a large argument as the program's first launch is recorded a second time, cut along the batch
    into parts that the runtime issues while the rest of the argument is still being uploaded. Whole calls (parts) give
    the bits of the same program replayed on resident inputs (the launch as recorded), call after call with new
    images; the oracle agrees on a slice of the batch; programs whose first launch does not qualify record no parts.'''
    rng = np.random.default_rng(41)
    lax, nn = mj.lax, mj.nn
    def stem(params, x):
        y = lax.conv_general_dilated(x, params['w'], (2, 2), ((3, 3), (3, 3)), dimension_numbers=W.NHWC)
        y = nn.relu(nn.batch_norm_inference(y, params['g'], params['b'], params['m'], params['v']))
        return y.reshape(x.shape[0], -1, 16).mean(axis=1), y[:, ::37, ::41, :]
    def frozen(a):
        a.flags.writeable = False
        return a
    params = dict(w=frozen((rng.standard_normal((7, 7, 3, 16)) / 12).astype(np.float32)), g=frozen(rng.random(16, dtype=np.float32) + 0.5),
                  b=frozen(rng.standard_normal(16).astype(np.float32)), m=frozen(rng.standard_normal(16).astype(np.float32)),
                  v=frozen(rng.random(16, dtype=np.float32) + 0.5))
    fn = vkjax_amd.wrap(stem, frontend='minijax')
    images = [rng.standard_normal((32, 224, 224, 3)).astype(np.float32) for _ in range(3)]
    results = [fn(params, x) for x in images]                       #(the first call uploads the parameters too, in front of x)
    interp = list(fn._jaxpr_interpreters.values())[0]
    assert len(interp.early_parts) == 4 and all(p.kernel == interp.launches[0].kernel for p, _, _ in interp.early_parts)
    assert [needed for _, _, needed in interp.early_parts] == [(k + 1) * images[0].nbytes // 4 for k in range(4)]
    for x, got in zip(images, results):
        interp.upload_inputs(params, x)
        interp.replay(1)
        mean, samples = interp.read_outputs()
        assert np.array_equal(np.asarray(got[0]).reshape(-1), mean.reshape(-1)) and np.array_equal(np.asarray(got[1]).reshape(-1), samples.reshape(-1))
    expected, _ = oracle_outputs(stem, [params, images[2][:2]])
    assert np.allclose(results[2][0][:2], expected[0], rtol=1e-4, atol=1e-5) and np.allclose(results[2][1][:2], expected[1], rtol=1e-4, atol=1e-5)
    #the general kernels: 1x1 and padded 3x3 convolutions whose parts run the whole launch's kernel (images are independent
    #of each other, and a wave adds up its contraction in one order whatever tile it works on)
    def conv_then_mean(w, b, x, padding):
        z = nn.relu(lax.conv_general_dilated(x, w, (1, 1), padding, dimension_numbers=W.NHWC) + b)
        return z.mean(axis=(1, 2)), z[:, ::29, ::31, :]
    with_parts = 0
    for shape, cout, k, padding in (((32, 64, 64, 64), 32, 1, 'VALID'), ((8, 128, 128, 64), 64, 1, 'VALID'), ((8, 128, 128, 64), 64, 3, 'SAME'),
                                    ((16, 96, 96, 32), 64, 3, 'SAME')):
        print(f'case: first launch in parts, {k}x{k} convolution over {shape} to {cout} features', flush=True)
        w, b = frozen((rng.standard_normal((k, k, shape[3], cout)) / 8).astype(np.float32)), frozen(rng.standard_normal(cout).astype(np.float32))
        g = vkjax_amd.wrap(lambda w, b, x: conv_then_mean(w, b, x, padding), frontend='minijax')
        xs = [rng.standard_normal(shape).astype(np.float32) for _ in range(2)]
        got = [g(w, b, x) for x in xs]
        interp = list(g._jaxpr_interpreters.values())[0]
        with_parts += bool(interp.early_parts)
        for x, (mean, samples) in zip(xs, got):
            interp.upload_inputs(w, b, x)
            interp.replay(1)
            whole = interp.read_outputs()
            assert np.array_equal(np.asarray(mean).reshape(-1), whole[0].reshape(-1)) and np.array_equal(np.asarray(samples).reshape(-1), whole[1].reshape(-1))
        expected, _ = oracle_outputs(lambda w, b, x: conv_then_mean(w, b, x, padding), [w, b, xs[1][:1]])
        assert np.allclose(got[1][0][:1], expected[0], rtol=1e-4, atol=1e-5) and np.allclose(got[1][1][:1], expected[1], rtol=1e-4, atol=1e-5)
    assert with_parts >= 2
    #a first launch that is no convolution over a large argument, or one in the mixed tiling: no parts
    small = vkjax_amd.wrap(stem, frontend='minijax')
    small(params, images[0][:4])
    assert list(small._jaxpr_interpreters.values())[0].early_parts == []
    fn2 = vkjax_amd.wrap(lambda x: nn.relu(x) * 2.0, frontend='minijax')
    big = rng.standard_normal((1 << 23,)).astype(np.float32)
    assert np.array_equal(fn2(big), np.maximum(big, 0) * 2.0) and list(fn2._jaxpr_interpreters.values())[0].early_parts == []
