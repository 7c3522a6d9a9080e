"""Persistent key/value store behind `Compiler.compile_cached`: one sqlite file, one table per cache key.

Mirrors env.disk_get / env.disk_put of the reference (/root/reference/jsgrad/env/node.ts:89-122) and its paths
(/root/reference/jsgrad/env/web.ts:26-31): `$CACHE_DB`, else `$CACHE_DIR|$XDG_CACHE_HOME|~/.cache` + `/jsgrad/jsgrad.db`;
tables are named `<table>_<DB_VERSION>`; a failing store never fails the caller (the value is simply compiled again).
"""
from __future__ import annotations

import os
import sqlite3

DB_VERSION = 1


def cache_dir() -> str:
    root = os.environ.get("CACHE_DIR") or os.environ.get("XDG_CACHE_HOME") or os.path.join(os.path.expanduser("~"), ".cache")
    return os.path.join(root, "jsgrad")


def cache_db() -> str:
    return os.environ.get("CACHE_DB") or os.path.join(cache_dir(), "jsgrad.db")


_conn: dict[str, sqlite3.Connection] = {}
_tables: set[tuple[str, str]] = set()


def _db() -> sqlite3.Connection:
    path = cache_db()
    if path not in _conn:
        os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
        _conn[path] = sqlite3.connect(path, timeout=30.0)
    return _conn[path]


def _name(table: str) -> str:
    return f"{table}_{DB_VERSION}"


def disk_get(table: str, key: str):
    try:
        row = _db().execute(f'SELECT value FROM "{_name(table)}" WHERE key = ?', (key,)).fetchone()
    except sqlite3.Error:
        return None
    return None if row is None else row[0]


def disk_put(table: str, key: str, value) -> None:
    if not isinstance(value, (str, bytes)):
        raise TypeError(f"Invalid value type {type(value).__name__}")
    try:
        db = _db()
        if (cache_db(), _name(table)) not in _tables:
            kind = "TEXT" if isinstance(value, str) else "BLOB"
            db.execute(f'CREATE TABLE IF NOT EXISTS "{_name(table)}" (key TEXT PRIMARY KEY, value {kind})')
            _tables.add((cache_db(), _name(table)))
        db.execute(f'INSERT OR REPLACE INTO "{_name(table)}" (key, value) VALUES (?, ?)', (key, value))
        db.commit()
    except sqlite3.Error as e:      # as in the reference: report, do not fail the compile
        import sys
        print(f"disk_put: {e}", file=sys.stderr)
