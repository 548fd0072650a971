"""Tuning records on disk: ``data_base/best_record.json`` and ``data_base/tuning_record.py``
(python/dtas/engine/database.py:10-51).  Same files, same keys (function name followed by the
bucket ranges; ``latency(ms)`` and ``config``); the reference's ``mod`` field held the scheduled TIR
script, here it holds the kernel variant's call-table row."""
from __future__ import annotations

import json
from typing import Tuple

from ..common.config import Range


class DataBase:
    def __init__(self, best_record_path: str, tuning_record_path: str):
        self.data = {}
        self.best_record_path = best_record_path
        self.tuning_record_path = tuning_record_path

    @staticmethod
    def _latency(cr):
        return None if cr.latency == float("inf") else cr.latency

    def commit_tuning_record(self, range_tuple: Tuple[Range, ...], cr) -> None:
        try:
            with open(self.tuning_record_path, "a") as f:
                lat = self._latency(cr)
                f.write(f"#name: {cr.name}\n#range: {range_tuple}  latency(ms): {lat if lat is not None else 'n/a'} \n")
                f.write(f"#config: {cr.config}\n")
                f.write(f"#call_table_row: {cr.abi.to_dict()}\n \n")
        except OSError:
            return

    def commit_best_record(self, range_tuple: Tuple[Range, ...], cr) -> None:
        key = cr.name
        for r in range_tuple:
            key += "_" + str(r)
        record = {key: {"latency(ms)": self._latency(cr), "config": [cr.config.to_dict()], "mod": cr.abi.to_dict()}}
        try:
            with open(self.best_record_path, "r") as f:
                data = json.load(f)
        except FileNotFoundError:
            data = []
        data.append(record)
        with open(self.best_record_path, "w") as f:
            f.write(json.dumps(data, indent=4))

    def save_to_file(self, filename: str) -> None:
        with open(filename, "w") as f:
            json.dump(self.data, f, indent=2)

    def load_from_file(self, filename: str) -> None:
        with open(filename, "r") as f:
            self.data = json.load(f)
