"""On-disk store of run-time compiled code objects.

Two kinds of files in one directory, both written with write-to-temp +
atomic rename so that concurrent processes never see a partial file:

* ``fn-<sha256(key)>.json``  function key -> {lowered_name, code_hash}
* ``code-<code_hash>.hsaco`` the code object itself (shared by every function
  that was compiled in the same program)

plus ``source_hash``, the hash of the device headers the entries were built
from.  When the headers change every entry is dropped, which is the
invalidation rule of the reference's LMDB store
(module_cache/cubin_database.py:46-67).
"""
from __future__ import annotations

import hashlib
import json
import os
import tempfile
from pathlib import Path
from typing import Optional, Tuple


class FunctionKey:
    """What a compiled function depends on (reference: function_db_key.py:3-28,
    plus the compiler flags, which the reference keeps constant)."""

    def __init__(self, package_name, package_version, toolchain_version, arch, flags, function_name):
        self.fields = {
            "package_name": package_name,
            "package_version": package_version,
            "toolchain_version": toolchain_version,
            "arch": arch,
            "flags": flags,
            "function_name": function_name,
        }

    def to_bytes(self) -> bytes:
        return json.dumps(self.fields, sort_keys=True).encode("utf-8")

    def digest(self) -> str:
        return hashlib.sha256(self.to_bytes()).hexdigest()

    def __repr__(self):
        return f"FunctionKey({self.fields})"


def _atomic_write(path: Path, data: bytes) -> None:
    fd, tmp = tempfile.mkstemp(dir=str(path.parent), prefix=path.name + ".", suffix=".tmp")
    try:
        with os.fdopen(fd, "wb") as f:
            f.write(data)
        os.replace(tmp, path)
    except BaseException:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise


class CodeObjectStore:
    def __init__(self, cache_dir: Path, source_hash: str, debug: bool = False):
        self.dir = Path(cache_dir)
        self.dir.mkdir(parents=True, exist_ok=True)
        self._check_source_hash(source_hash, debug)

    def _check_source_hash(self, source_hash: str, debug: bool) -> bool:
        marker = self.dir / "source_hash"
        stored = marker.read_text().strip() if marker.exists() else None
        cleared = False
        if stored is not None and stored != source_hash:
            if debug:
                print(f"(Kermac Debug) File source hash mismatch (stored: {stored}, provided: {source_hash}).")
                print("(Kermac Debug) Clearing store of pre-built code objects")
            for entry in self.dir.iterdir():
                if entry.name.startswith(("fn-", "code-")):
                    try:
                        entry.unlink()
                    except OSError:
                        pass
            cleared = True
        elif debug and stored is not None:
            print("(Kermac Debug) Hashes match. Keeping pre-built code objects.")
        if stored != source_hash:
            _atomic_write(marker, source_hash.encode())
        return cleared

    def get_function_mapping(self, key: FunctionKey) -> Optional[Tuple[str, str]]:
        path = self.dir / f"fn-{key.digest()}.json"
        try:
            record = json.loads(path.read_text())
        except (OSError, ValueError):
            return None
        if record.get("key") != key.fields:
            return None
        if not (self.dir / f"code-{record['code_hash']}.hsaco").exists():
            return None
        return record["lowered_name"], record["code_hash"]

    def put_function_mapping(self, key: FunctionKey, lowered_name: str, code_hash: str) -> None:
        record = {"key": key.fields, "lowered_name": lowered_name, "code_hash": code_hash}
        _atomic_write(self.dir / f"fn-{key.digest()}.json", json.dumps(record, sort_keys=True).encode())

    def put_code(self, code: bytes) -> str:
        code_hash = hashlib.sha256(code).hexdigest()
        path = self.dir / f"code-{code_hash}.hsaco"
        if not path.exists():
            _atomic_write(path, code)
        return code_hash

    def get_code(self, code_hash: str) -> Optional[bytes]:
        """The stored code object, or None when it is missing or its bytes no longer
        hash to its name (a truncated or edited file): the caller then recompiles."""
        path = self.dir / f"code-{code_hash}.hsaco"
        try:
            code = path.read_bytes()
        except OSError:
            return None
        if hashlib.sha256(code).hexdigest() != code_hash:
            try:
                path.unlink()
            except OSError:
                pass
            return None
        return code
