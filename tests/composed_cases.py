"""Models exercising the composed rules (clip, where, cumsum, amax / amin, prod) and the
extended scalar table; shared by the oracle, host-logic and GPU tests.  x has 12 entries."""

import numpy as np

MASK = np.array([True, False, True, True, False, False, True, False, True, True, False, True])


_OFFS = ((0.37 * np.arange(72)) % 2.9).astype(np.float32)
_SPREAD = np.random.default_rng(72).uniform(-2.0, 2.0, size=72).astype(np.float32)


_W1 = np.cos(np.arange(32, dtype=np.float32)).reshape(4, 8)
_W2 = np.sin(0.7 * np.arange(128, dtype=np.float32)).reshape(4, 4, 8)
_W3 = np.cos(1.3 * np.arange(16, dtype=np.float32)).reshape(4, 4)


def _g(xp, x, sl):
    return xp.getitem(x, (sl,))


CASES = {
    'clip': lambda xp, x: xp.clip(xp.multiply(xp.sin(x), 2.0), -0.7, 1.1),
    'where': lambda xp, x: xp.where(MASK, xp.sin(x), xp.multiply(x, x)),
    'where_const': lambda xp, x: xp.where(MASK, xp.tanh(x), 0.25),
    'cumsum': lambda xp, x: xp.cumsum(xp.tanh(x)),
    'cumsum_axis0': lambda xp, x: xp.cumsum(xp.reshape(xp.sin(x), (4, 3)), axis=0),
    'amax': lambda xp, x: xp.amax(xp.reshape(xp.sin(xp.multiply(x, 1.7)), (3, 4)), axis=-1),
    'amin_axis0': lambda xp, x: xp.amin(xp.reshape(xp.cos(xp.multiply(x, 1.3)), (3, 4)), axis=0),
    'prod': lambda xp, x: xp.prod(xp.reshape(xp.add(xp.sin(x), 1.5), (3, 4)), axis=-1),
    'scalar_table': lambda xp, x: xp.add(
        xp.add(xp.sinh(_g(xp, x, slice(0, 4))), xp.arctan(_g(xp, x, slice(4, 8)))),
        xp.multiply(xp.erf(_g(xp, x, slice(8, 12))), xp.power(xp.add(xp.square(_g(xp, x, slice(0, 4))), 0.5), 1.5))),
    'flip_pad': lambda xp, x: xp.pad(xp.flip(xp.reshape(xp.sin(x), (4, 3)), 0), ((1, 0), (0, 2)), 0.5),
    'where_data_dependent': lambda xp, x: xp.where(xp.greater(x, 0.1), xp.tanh(x), xp.multiply(xp.cos(x), 0.3)),
    'logaddexp': lambda xp, x: xp.logaddexp(_g(xp, x, slice(0, 6)), xp.sin(_g(xp, x, slice(6, 12)))),
    'cumprod': lambda xp, x: xp.cumprod(xp.reshape(xp.add(xp.sin(x), 1.5), (3, 4)), axis=-1),
    'cummax': lambda xp, x: xp.cummax(xp.reshape(xp.sin(xp.multiply(x, 1.9)), (3, 4)), axis=-1),
    'cummin_axis0': lambda xp, x: xp.cummin(xp.reshape(xp.cos(xp.multiply(x, 1.4)), (3, 4)), axis=0),
    # atan2 over all four quadrants and both half-plane branches (x = 12 seeded normals * 0.8)
    'atan2': lambda xp, x: xp.arctan2(xp.sin(xp.multiply(_g(xp, x, slice(0, 6)), 2.0)),
                                      xp.add(xp.cos(xp.multiply(_g(xp, x, slice(6, 12)), 3.0)), 0.1)),
    'atan2_const': lambda xp, x: xp.arctan2(xp.sin(x), -0.4),
    'pow_variable_exponent': lambda xp, x: xp.power(xp.add(xp.square(_g(xp, x, slice(0, 6))), 0.7),
                                                    xp.sin(_g(xp, x, slice(6, 12)))),
    'pow_constant_base': lambda xp, x: xp.power(1.7, xp.tanh(x)),
    'rem': lambda xp, x: xp.remainder(xp.multiply(x, 3.0), xp.add(xp.cos(x), 1.6)),
    'exp2': lambda xp, x: xp.exp2(xp.sin(x)),
    'split_stack_tile': lambda xp, x: xp.tile(xp.stack([xp.multiply(a, b) for a, b in zip(
        xp.split(xp.sin(x), 2), xp.split(xp.tanh(x), [6]))], axis=1), (2, 1)),
    'dynamic_slices': lambda xp, x: xp.dynamic_update_slice(
        xp.reshape(xp.sin(x), (3, 4)), xp.dynamic_slice(xp.reshape(xp.square(x), (3, 4)), (1, 2), (2, 2)), (0, 1)),
    # fused exponential envelope: dense input, and (in the host / GPU tests with a threshold) sparse
    'exp_envelope': lambda xp, x: xp.exp_envelope(
        xp.add(xp.square(xp.reshape(x, (4, 3))), 0.3),
        np.linspace(0.4, 1.6, 24, dtype=np.float32).reshape(3, 8), np.cos(np.arange(24, dtype=np.float32)).reshape(3, 8)),
    'exp_envelope_mixed_rows': lambda xp, x: xp.exp_envelope(
        xp.reshape(xp.add(xp.square(xp.dot(xp.reshape(x, (4, 3)), np.ones((3, 3), dtype=np.float32))), 0.3), (4, 3)),
        np.linspace(0.4, 1.6, 12, dtype=np.float32).reshape(3, 4), np.cos(np.arange(12, dtype=np.float32)).reshape(3, 4)),
    # reduced / scanned axes longer than 64 entries (72 and an odd 65): tree folds and log-depth scans
    # (tanh of a spread of arguments: at the largest entry the derivative is not near a zero of its own, as it
    # would be at the top of a sine, where float32 argument rounding decides the Jacobian's relative error)
    'amax_long_axis': lambda xp, x: xp.amax(xp.tanh(xp.multiply(xp.add(xp.tile(x, (6,)), _SPREAD), 0.3)), axis=-1),
    'prod_long_odd_axis': lambda xp, x: xp.prod(
        xp.add(xp.multiply(xp.sin(_g(xp, xp.add(xp.tile(x, (6,)), _OFFS), slice(0, 65))), 0.2), 1.0), axis=-1),
    'cumprod_long_axis': lambda xp, x: xp.cumprod(xp.add(xp.multiply(xp.sin(xp.add(xp.tile(x, (6,)), _OFFS)), 0.2), 1.0)),
    'cummax_long_axis': lambda xp, x: xp.cummax(xp.tanh(xp.multiply(xp.add(xp.tile(x, (6,)), _SPREAD), 0.3))),
    # jax.lax.pad as the reference's tests use it (test/test_layers.py:668-682): interior padding, a padding value
    # that depends on the input, negative (cropping) edges
    'lax_pad_interior': lambda xp, x: xp.lax_pad(xp.reshape(xp.sin(x), (4, 3)), 7.0, ((1, 0, 1), (0, 2, 0))),
    'lax_pad_varying_value': lambda xp, x: xp.lax_pad(xp.tanh(_g(xp, x, slice(0, 11))),
                                                       xp.square(xp.reshape(_g(xp, x, slice(11, 12)), ())), ((2, 1, 1),)),
    'lax_pad_negative': lambda xp, x: xp.lax_pad(xp.multiply(xp.sin(x), x), 0.0, ((-1, -2, 0),)),
    'lax_pad_negative_interior': lambda xp, x: xp.lax_pad(xp.reshape(xp.cos(x), (3, 4)), -1.5, ((-1, 2, 2), (1, -3, 1))),
    # jax.numpy / jax.nn names that the reference reaches through its tracer (test/test_layers.py:695-716 uses the erf
    # form of gelu); here they are compositions of the rules
    'activations_by_name': lambda xp, x: xp.add(
        xp.add(xp.gelu(_g(xp, x, slice(0, 4)), approximate=False), xp.gelu(_g(xp, x, slice(4, 8)))),
        xp.add(xp.elu(xp.multiply(_g(xp, x, slice(8, 12)), 2.0), 1.3),
               xp.add(xp.relu(xp.sin(xp.multiply(_g(xp, x, slice(0, 4)), 3.0))), xp.leaky_relu(_g(xp, x, slice(4, 8)), 0.2)))),
    'log_softmax_var_std': lambda xp, x: xp.add(
        xp.sum(xp.log_softmax(xp.reshape(xp.sin(x), (3, 4)), axis=-1), axis=0),
        xp.add(xp.var(xp.reshape(xp.tanh(x), (3, 4)), axis=0),
               xp.reshape(xp.std(xp.reshape(xp.multiply(x, x), (4, 3)), axis=-1, keepdims=True), (4,)))),
    'norm_vdot_outer': lambda xp, x: xp.multiply(
        xp.outer(xp.sin(_g(xp, x, slice(0, 3))), xp.tanh(_g(xp, x, slice(3, 7)))),
        xp.add(xp.norm(xp.reshape(x, (3, 4)), axis=0), xp.vdot(xp.cos(x), xp.reshape(xp.square(x), (3, 4))))),
    'tensordot_inner': lambda xp, x: xp.add(
        xp.tensordot(xp.reshape(xp.sin(x), (2, 3, 2)), xp.reshape(xp.tanh(x), (3, 2, 2)), axes=2),
        xp.inner(xp.reshape(xp.cos(x), (2, 6)), np.linspace(-1.0, 1.0, 12, dtype=np.float32).reshape(2, 6))),
    'moveaxis_take_roll_repeat': lambda xp, x: xp.add(
        xp.take(xp.moveaxis(xp.reshape(xp.sin(x), (2, 3, 2)), 0, -1), np.array([[2, 0], [1, 1]]), axis=0),
        xp.reshape(xp.take(xp.roll(xp.repeat(xp.tanh(x), 2, axis=0), 5, axis=0), np.arange(0, 24, 3)), (2, 2, 2))),
    'diagonal_trace': lambda xp, x: xp.add(
        xp.diagonal(xp.reshape(xp.sin(x), (3, 2, 2))), xp.reshape(xp.trace(xp.reshape(xp.multiply(x, x), (3, 2, 2)), offset=1), (3, 1))),
    # einsum with three operands, an ellipsis and the implicit output form (test/test_layers.py:255-262:
    # dot(x, w1) + einsum('...i,...j,...ijk->...k', x, x, w2)); constants and triplets mixed
    'einsum_three_operands': lambda xp, x: xp.add(
        xp.dot(xp.reshape(x, (3, 4)), _W1),
        xp.einsum('...i,...j,...ijk->...k', xp.reshape(xp.sin(x), (3, 4)), xp.reshape(x, (3, 4)), _W2)),
    'einsum_implicit_and_chain': lambda xp, x: xp.add(
        xp.einsum('ij,jk', xp.reshape(xp.sin(x), (3, 4)), xp.reshape(xp.tanh(x), (4, 3))),
        xp.einsum('ai,ij,bj->ab', xp.reshape(xp.cos(x), (3, 4)), _W3, xp.reshape(xp.multiply(x, x), (3, 4)))),
    'inverse_trig': lambda xp, x: xp.add(xp.arcsin(xp.multiply(xp.tanh(x), 0.9)),
                                         xp.arccosh(xp.add(xp.square(x), 1.2))),
}
