"""Registers-per-thread look-up for a kernel on another architecture.

Same contract as analyzer/habitat/analysis/wave_scaling/metadata.py:7-44: a
sqlite table kernels(name, arch, registers_per_thread); the entry with the
largest arch not above the device's is used; None when there is none.
`NullMetadataManager` is the manager to use without a table.
"""
import logging
import sqlite3

logger = logging.getLogger(__name__)

_QUERY = ("SELECT arch, registers_per_thread FROM kernels "
          "WHERE name = ? AND arch <= ? ORDER BY arch DESC LIMIT 1")


def device_arch(device):
    """(7, 0) -> 70."""
    return int("".join(str(x) for x in device.compute_capability))


class MetadataManager:
    def __init__(self, path_to_lut):
        self._connection = sqlite3.connect(path_to_lut)

    def kernel_registers_for(self, kernel, device):
        arch = device_arch(device)
        row = self._connection.cursor().execute(_QUERY, (kernel.name, arch)).fetchone()
        if row is None:
            logger.debug('Missing kernel metadata entry for "%s" on arch %d.', kernel.name, arch)
            return None
        actual_arch, registers_per_thread = row
        if actual_arch != arch:
            logger.debug('Using substitute entry for "%s" at arch %d instead of %d.',
                         kernel.name, actual_arch, arch)
        return registers_per_thread

    def registers_for_names(self, names, device):
        """One look-up per distinct name; a list aligned with `names` (-1 = none)."""
        arch = device_arch(device)
        cur = self._connection.cursor()
        cache = {}
        out = []
        for name in names:
            if name not in cache:
                row = cur.execute(_QUERY, (name, arch)).fetchone()
                cache[name] = -1 if row is None else int(row[1])
            out.append(cache[name])
        return out


class NullMetadataManager:
    """No table: every kernel keeps its own register count."""

    def kernel_registers_for(self, kernel, device):
        return None

    def registers_for_names(self, names, device):
        return [-1] * len(names)
