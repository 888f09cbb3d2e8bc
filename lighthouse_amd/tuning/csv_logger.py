"""Row logger of the tuning runs (the role of examples/xegpu/csv_logger.py:6-52): the first row
fixes the columns, every row is echoed and appended to a file whose name is made unique."""

from __future__ import annotations

import csv
import os
import sys


class CSVLogger:
    def __init__(self, filename: str | None = None, echo_stdout: bool = True):
        self.filename = self._unique(filename) if filename else None
        self.echo_stdout = echo_stdout
        self.fieldnames: list[str] | None = None

    @staticmethod
    def _unique(path: str) -> str:
        base, ext = os.path.splitext(path)
        candidate, i = path, 1
        while os.path.exists(candidate):
            candidate = f"{base}_{i}{ext}"
            i += 1
        return candidate

    def log(self, data: dict) -> None:
        first = self.fieldnames is None
        if first:
            self.fieldnames = list(data.keys())
        missing = [k for k in self.fieldnames if k not in data]
        if missing:
            raise ValueError(f"row lacks columns {missing}")
        if self.echo_stdout:
            if first:
                print(",".join(self.fieldnames), file=sys.stdout)
            print(",".join(str(data[k]) for k in self.fieldnames), file=sys.stdout)
        if self.filename is not None:
            with open(self.filename, "a", newline="") as f:
                writer = csv.DictWriter(f, fieldnames=self.fieldnames, extrasaction="ignore")
                if first:
                    writer.writeheader()
                writer.writerow(data)
