"""Helper of the tests that need npz archives at the size of real expert files: writes an archive through Python's
zipfile (as numpy.savez does, stored members, zip64 local headers) onto a file object that turns long runs of
zero bytes into holes, so that a 4.4 GB archive whose large members are zeros costs neither the time nor the
disk space of its size.  The archive's structure - zip64 extra fields, offsets beyond 4 GiB, the zip64 end record
and its locator - is exactly what zipfile writes for a file of that size."""
import zipfile

import numpy as np


class HoleyFile:
    """A binary file for writing in which a block of zeros of a MiB or more becomes a seek: the filesystem
    stores a hole, and reads return zeros."""

    def __init__(self, path):
        self.f = open(path, "wb")

    def write(self, data):
        n = len(data)
        if n >= (1 << 20) and not any(memoryview(data)[:4096]) and data.count(0) == n:
            self.f.seek(n, 1)
        else:
            self.f.write(data)
        return n

    def tell(self):
        return self.f.tell()

    def seek(self, *a):
        return self.f.seek(*a)

    def flush(self):
        self.f.flush()

    def close(self):
        self.f.truncate(max(self.f.tell(), self.f.seek(0, 2)))
        self.f.close()

    # zipfile probes these
    def seekable(self):
        return True

    def writable(self):
        return True


def npy_header(shape, fortran_order=False):
    import io
    buf = io.BytesIO()
    np.lib.format.write_array_header_1_0(buf, {"descr": "<f4", "fortran_order": fortran_order, "shape": tuple(shape)})
    return buf.getvalue()


def write_npz(path, members):
    """members: iterable of (name, array or shape).  An array is written as numpy would; a bare shape stands for a
    float32 array of zeros of that shape, written as a hole."""
    hf = HoleyFile(path)
    zeros = bytes(64 << 20)
    with zipfile.ZipFile(hf, "w", zipfile.ZIP_STORED, allowZip64=True) as z:
        for name, a in members:
            with z.open(name + ".npy", "w", force_zip64=True) as m:  # as numpy.savez opens its members
                if isinstance(a, np.ndarray):
                    a = np.ascontiguousarray(a, np.float32)
                    m.write(npy_header(a.shape))
                    m.write(a.tobytes())
                else:
                    m.write(npy_header(a))
                    left = 4 * int(np.prod(a))
                    while left > 0:
                        n = min(left, len(zeros))
                        m.write(zeros[:n] if n < len(zeros) else zeros)
                        left -= n
    hf.close()
