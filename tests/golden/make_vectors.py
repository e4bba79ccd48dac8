'''Writes tests/golden/known_answers.json.

Every value in that file is a PUBLISHED known answer, typed in here from its source, not
something computed by this repository's code:
  * Threefry-2x32-20 known-answer vectors of the Random123 distribution (kat_vectors), the same
    three that JAX's own test-suite checks (tests/random_test.py, testThreefry2x32).
  * `jax.random.split(jax.random.PRNGKey(0))` and `jax.random.uniform(jax.random.PRNGKey(0))`
    as printed in the JAX documentation ("Pseudo random numbers in JAX") for the original,
    non-partitionable threefry layout.
  * `jax.random.normal(PRNGKey(0), (1,))` = [-0.20584226] (JAX documentation, "JAX PRNG design") and the ten
    values `random.normal(random.PRNGKey(0), (10,))` prints in the JAX quickstart; `uniform(key(0))` = 0.947667
    and `uniform(split(key(0))[1])` = 0.00729382 from the jax.random module documentation (partitionable layout).
  * The literal expectations of the reference's own tests: f(65) == 66, f(-5) == -4
    (tests/test_function.py:15-16), shift_right_logical(1, 32) == 0 (tests/test_basic_ops.py:150-151,305),
    buffer-reuse counts 2 and 8 (tests/test_bufferpool.py:40,63).
Run:  python tests/golden/make_vectors.py
'''
import json
import os

KNOWN = {
    'threefry2x32_kat': [
        {'key': ['0x00000000', '0x00000000'], 'counter': ['0x00000000', '0x00000000'], 'expected': ['0x6b200159', '0x99ba4efe']},
        {'key': ['0xffffffff', '0xffffffff'], 'counter': ['0xffffffff', '0xffffffff'], 'expected': ['0x1cb996fc', '0xbb002be7']},
        {'key': ['0x13198a2e', '0x03707344'], 'counter': ['0x243f6a88', '0x85a308d3'], 'expected': ['0xc4923a9c', '0x483df7a0']},
    ],
    'jax_random_split_PRNGKey0': [[4146024105, 967050713], [2718843009, 1272950319]],
    'jax_random_uniform_PRNGKey0': {'bits': 1797259609, 'value': 0.41845703},
    'jax_random_normal_PRNGKey0': {'shape_1': [-0.20584226],
                                   'shape_10': [-0.3721109, 0.26423115, -0.18252768, -0.7368197, -0.44030377, -0.1521442,
                                                -0.67135346, -0.5908641, 0.73168886, 0.5673026]},
    'jax_random_partitionable_key0': {'uniform': 0.947667, 'uniform_of_second_subkey': 0.00729382},
    'reference_test_literals': {'func0_65': 66, 'func0_minus5': -4, 'shift_right_logical_1_32': 0,
                                'bufferpool_lowlevel_unique_tensors': 2, 'bufferpool_highlevel_unique_tensors': 8,
                                'bufferpool_lowlevel_accesses': [[0, 2], [1], [3]]},
}

if __name__ == '__main__':
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'known_answers.json')
    with open(path, 'w') as f:
        json.dump(KNOWN, f, indent=1)
    print('wrote', path)
