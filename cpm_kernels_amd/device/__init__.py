"""Device bookkeeping with the reference's names (cpm_kernels/device/__init__.py:106-158):
``Device``, ``current_device()``, ``num_devices()``, ``Device.architecture``, ``Device.use()``.

The reference caches 101 cudaDevAttr* values per device and creates a cuBLASLt handle in
``use()``.  The HIP kernels are statically linked into one library and need no handle, so a
device here is its ordinal plus the properties the path and its roofline use.
"""
from ..library import cpmk


class _Device:
    def __init__(self, index: int):
        self._index = index
        self.attributes = cpmk.device_props(index)

    def use(self):
        cpmk.set_device(self._index)


def _enumerate():
    if cpmk.version <= 0:
        return []
    try:
        return [_Device(i) for i in range(cpmk.device_count())]
    except RuntimeError:       # no GPU / no driver on this host
        return []


_DEVICES = _enumerate()


class Device:
    def __init__(self, index: int) -> None:
        # (the reference tests `index > len`, an off-by-one; a bad index raises here)
        if index < 0 or index >= len(_DEVICES):
            raise ValueError("Device index out of range (%d >= %d)" % (index, len(_DEVICES)))
        self._device = _DEVICES[index]
        self.index = index
        for kw, value in self._device.attributes.items():
            setattr(self, kw, value)

    def attr(self, name: str):
        return self._device.attributes[name]

    @property
    def architecture(self) -> int:
        """Numeric part of the gfx target (gfx950 -> 950); the reference returns the CUDA
        compute capability major*10+minor here."""
        digits = "".join(c for c in self._device.attributes["name"][3:] if c.isalnum())
        try:
            return int(digits, 16) if any(c in "abcdef" for c in digits) else int(digits)
        except ValueError:
            return 0

    def use(self):
        self._device.use()


def num_devices() -> int:
    return len(_DEVICES)


def current_device() -> Device:
    return Device(cpmk.get_device())
