"""Gradient-table generator: forward table -> difference-based gradient tables (int16, slope x 16).

Counterpart of the reference's ``scripts/gen_bp_lut.py`` with the same command line and the same output
file format, computed with vectorised NumPy instead of per-entry Python loops:

    python gen_bp_lut.py -f <..._lutfp.txt> -w <half window>  >  <..._lutfp+bp_avg_w_w.txt>

Definition (N = 2^bits, h = half window, F = forward table, float32 arithmetic as in the reference):
  S_a[a][b] = mean(F[max(0,a-h) : min(N,a+h+1), b]);    S_b likewise along b        (``gen_bp_lut.py:7-16,36-45``)
  interior  h+1 <= a <= N-h-2 :  g_a = (S_a[a+1][b] - S_a[a-1][b]) / 2              (``:54-55``)
  border                      :  g_a = (max - min of ROW b of F) / N   -- the reference indexes
                                 ``lut[0:N][b]``, i.e. row b, for the first operand (``:58-61``)
  g_b symmetric, its border rule uses row a (``:25-32``);   stored value = round-half-even(16 * g).
"""
import optparse
import sys

import numpy as np

HEADER_FWD = 'LUT for approximate multiplier:'
HEADER_GA = 'LUT for the gradient of the approximate multiplier w.r.t. the first operand:'
HEADER_GB = 'LUT for the gradient of the approximate multiplier w.r.t. the second operand:'


def _window_mean(F32, h, axis):
    """Moving average with a window clipped at the table edge; float32 like ``np.mean`` of float32 data:
    window sums are exact integers (< 2^24 for 16-bit entries and windows up to 256) and the division is
    one float32 operation."""
    n = F32.shape[axis]
    c = np.cumsum(F32.astype(np.int64), axis=axis)
    c = np.concatenate([np.zeros_like(np.take(c, [0], axis=axis)), c], axis=axis)
    idx = np.arange(n)
    lo, hi = np.maximum(0, idx - h), np.minimum(n, idx + h + 1)
    sums = np.take(c, hi, axis=axis) - np.take(c, lo, axis=axis)
    cnt = (hi - lo).astype(np.float32)
    shape = [1, 1]
    shape[axis] = n
    return (sums.astype(np.float32) / cnt.reshape(shape)).astype(np.float32)


def gradient_tables(fwd, half_ws, rounded=True):
    """fwd: (N, N) integer table.  Returns (grad_a16, grad_b16) int64 = round(16 * slope), the encoding of the reference's
    table files; rounded=False returns the float32 slopes themselves (for the float-table backward pass)."""
    assert half_ws >= 1
    F32 = np.asarray(fwd).astype(np.float32)
    n = F32.shape[0]
    # np.mean over float32 accumulates pairwise in float32; for integer data whose window sums stay below
    # 2^24 every partial sum is exact, so the exact integer sum divided once reproduces it bit for bit
    assert float(F32.max()) * (2 * half_ws + 1) < 2 ** 24, "window sums would not be exact in float32"
    sa = _window_mean(F32, half_ws, 0)
    sb = _window_mean(F32, half_ws, 1)
    row_range = (F32.max(axis=1) - F32.min(axis=1)) / np.float32(n)      # per row r: (max - min of F[r, :]) / N
    ga = np.empty_like(F32)
    gb = np.empty_like(F32)
    ga[:, :] = row_range[None, :]            # border rule of the first operand: row b (reference quirk)
    gb[:, :] = row_range[:, None]            # border rule of the second operand: row a
    lo, hi = half_ws + 1, n - half_ws - 2    # inclusive interior range
    if hi >= lo:
        ga[lo:hi + 1, :] = (sa[lo + 1:hi + 2, :] - sa[lo - 1:hi, :]) / np.float32(2)
        gb[:, lo:hi + 1] = (sb[:, lo + 1:hi + 2] - sb[:, lo - 1:hi]) / np.float32(2)
    if not rounded:
        return ga, gb
    return (np.round(ga * np.float32(16.0)).astype(np.int64), np.round(gb * np.float32(16.0)).astype(np.int64))


def bits_from_name(file_name):
    for bits in (8, 7, 4, 6):
        if file_name.find(f'mul{bits}') != -1 or file_name.find(f'{bits}_{bits}') != -1:
            return bits
    raise ValueError('Unknown bit width')


def read_forward_table(file_name, bits):
    n = 1 << bits
    lines = open(file_name).read().splitlines()
    start = next(i for i, l in enumerate(lines) if l.startswith(HEADER_FWD))
    vals = np.array(' '.join(lines[start + 1:start + 1 + n * n]).split(), dtype=np.int64).reshape(-1, 3)
    table = np.zeros((n, n), np.int64)
    table[vals[:, 0], vals[:, 1]] = vals[:, 2]
    return table


def write_tables(out, fwd, ga16, gb16):
    n = fwd.shape[0]
    a, b = np.divmod(np.arange(n * n), n)
    for header, tab, lo, hi in ((HEADER_FWD, fwd, 0, 2 ** 16), (HEADER_GA, ga16, -2 ** 15, 2 ** 15), (HEADER_GB, gb16, -2 ** 15, 2 ** 15)):
        assert tab.min() >= lo and tab.max() < hi, 'table value out of range'
        out.write(header + '\n')
        out.write('\n'.join(f'{x} {y} {v}' for x, y, v in zip(a, b, tab.ravel())) + '\n')


def main(argv=None):
    parser = optparse.OptionParser()
    parser.add_option('-f', '--file', dest='file_name', help='file name of the lookup table', default=None)
    parser.add_option('-w', '--half_ws_a', dest='half_ws_a', help='half window size for smoothing', default=32)
    options, _ = parser.parse_args(argv)
    half_ws = int(options.half_ws_a)
    bits = bits_from_name(options.file_name)
    fwd = read_forward_table(options.file_name, bits)
    ga16, gb16 = gradient_tables(fwd, half_ws)
    exact = np.arange(1 << bits)[:, None] * np.arange(1 << bits)[None, :]
    err = np.abs(fwd - exact)
    print(f'INFO: file_name={options.file_name}, half_ws_a={half_ws}, half_ws_b={half_ws}, QUANTIZATION_BIT={bits}')
    print(f'INFO: Error rate between lut_appmult and lut_mult: {np.mean(fwd != exact) * 100}%')
    print(f'INFO: Mean error distance between lut_appmult and lut_mult: {err.mean()}')
    print(f'INFO: Maximum error distance between lut_appmult and lut_mult: {err.max()}')
    write_tables(sys.stdout, fwd, ga16, gb16)


if __name__ == '__main__':
    main()
