"""`delayrepay.random`: backend random routines wrapped as lazy leaves
(cf. delayrepay/random.py:6-13), and an opt-in generator that runs on the device.

`rand`, `randn`, `random`, `randint`, `choice`, `seed` are the reference's surface: the
legacy global NumPy stream, drawn on the host and uploaded, so a seeded program sees the
numbers it always saw.  `device(seed)` returns a `DeviceRandom`: Philox-4x64-10, the
counter-based generator of `numpy.random.Philox`, evaluated inside the fused kernels from
the element index.  Its arrays are lazy; used in a 1-d expression of their own length
they cost no memory traffic at all, and they hold exactly the numbers
`numpy.random.Generator(numpy.random.Philox(key=seed))` hands out, call after call, on
either backend.
"""
import numpy

from . import backend as be
from .delayarray import RandEx, cast, concatenate

_rnd = be.backend.np.random

rand = cast(_rnd.rand)
randn = cast(_rnd.randn)
random = cast(_rnd.random)
randint = cast(_rnd.randint)
choice = cast(_rnd.choice)
seed = _rnd.seed


class DeviceRandom:
    """Philox-4x64-10 stream with the 128-bit key `seed` and the 256-bit start counter
    `counter`; the same numbers as `numpy.random.Generator(numpy.random.Philox(key=seed,
    counter=counter))` in the same order (one 64-bit output per number drawn)."""

    def __init__(self, seed=0, counter=0):
        seed, counter = int(seed), int(counter)
        if not 0 <= seed < 1 << 128:
            raise ValueError("the key of a Philox stream is an integer in [0, 2**128)")
        if not 0 <= counter < 1 << 256:
            raise ValueError("the counter of a Philox stream is an integer in [0, 2**256)")
        self.key = seed
        # NumPy steps the counter before it makes the first block
        self._first = (counter + 1) % (1 << 256)
        self.pos = 0           # outputs handed out so far
        self._half = None      # the output whose high half the next float32 takes first

    def _draw(self, size, dtype):
        shape = () if size is None else ((int(size),) if isinstance(size, (int, numpy.integer))
                                         else tuple(int(d) for d in size))
        n = 1
        for d in shape:
            n *= d
        first, pos = divmod(self.pos, 4)
        node = RandEx(n, self.key, (self._first + first) % (1 << 256), pos, dtype)
        self.pos += n
        if len(shape) == 1:
            return node
        return node.reshape(shape) if shape else node.reshape(1)[0]

    def random_raw(self, size=None):
        """Raw 64-bit outputs as int64 (view them as uint64 to compare with NumPy)."""
        return self._draw(size, numpy.int64)

    def random(self, size=None, dtype=numpy.float64):
        """Numbers in [0, 1), as `Generator.random`: doubles, or with `dtype=float32`
        floats, two from every output of the stream."""
        if numpy.dtype(dtype) == numpy.float32:
            return self._draw_floats(size)
        if numpy.dtype(dtype) != numpy.float64:
            raise TypeError("random() makes float64 or float32 numbers")
        return self._draw(size, numpy.float64)

    def _draw_floats(self, size):
        """NumPy hands the low half of an output to one float and keeps the high half for
        the next float that is asked for, whatever is drawn in between."""
        shape = () if size is None else ((int(size),) if isinstance(size, (int, numpy.integer))
                                         else tuple(int(d) for d in size))
        n = 1
        for d in shape:
            n *= d
        parts = []
        left = n
        if self._half is not None and left:
            block, word = divmod(self._half, 4)
            parts.append(RandEx(1, self.key, (self._first + block) % (1 << 256), 2 * word + 1, numpy.float32))
            self._half = None
            left -= 1
        if left:
            block, word = divmod(self.pos, 4)
            parts.append(RandEx(left, self.key, (self._first + block) % (1 << 256), 2 * word, numpy.float32))
            if left % 2:
                self._half = self.pos + left // 2
            self.pos += (left + 1) // 2
        if not parts:
            node = RandEx(0, self.key, self._first, 0, numpy.float32)
        elif len(parts) == 1:
            node = parts[0]
        else:
            node = concatenate(parts)
        if len(shape) == 1:
            return node
        return node.reshape(shape) if shape else node.reshape(1)[0]

    def uniform(self, low=0.0, high=1.0, size=None):
        """`low + (high - low) * random()`, the arithmetic of `Generator.uniform`."""
        low, high = float(low), float(high)
        return low + (high - low) * self._draw(size, numpy.float64)


def device(seed=0, counter=0):
    """A generator whose numbers are made on the device (see the module docstring)."""
    return DeviceRandom(seed, counter)
