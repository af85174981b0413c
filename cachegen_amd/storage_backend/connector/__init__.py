"""Connectors to the store behind the remote backend
(LMCache/lmcache/storage_backend/connector/ in the reference).

A connector moves opaque byte strings under string keys.  "mem://name:0" is an in-process
store shared by every connector opened with the same name: it stands in for a server in tests
and single-process use.  "redis://host:port" needs the `redis` package at the time it is
opened.  The reference's own "lm://" server protocol is not provided."""
import abc
import re
import threading
from typing import Dict, List, Optional


class RemoteConnector(metaclass=abc.ABCMeta):
    """base_connector.py:9-62: exists / get / set / list over byte strings."""

    @abc.abstractmethod
    def exists(self, key: str) -> bool:
        raise NotImplementedError

    @abc.abstractmethod
    def get(self, key: str) -> Optional[bytes]:
        raise NotImplementedError

    @abc.abstractmethod
    def set(self, key: str, obj: bytes) -> None:
        raise NotImplementedError

    @abc.abstractmethod
    def list(self) -> List[str]:
        raise NotImplementedError


class InMemoryConnector(RemoteConnector):
    _stores: Dict[str, Dict[str, bytes]] = {}
    _lock = threading.Lock()

    def __init__(self, name: str):
        with InMemoryConnector._lock:
            self.store = InMemoryConnector._stores.setdefault(name, {})

    def exists(self, key):
        return key in self.store

    def get(self, key):
        return self.store.get(key, None)

    def set(self, key, obj):
        self.store[key] = bytes(obj)

    def list(self):
        return list(self.store.keys())

    @staticmethod
    def drop(name: str) -> None:
        """Forget the named store (tests)."""
        with InMemoryConnector._lock:
            InMemoryConnector._stores.pop(name, None)


class RedisConnector(RemoteConnector):
    """redis_connector.py:8-29: one Redis connection; keys are listed with SCAN."""

    def __init__(self, host: str, port: int):
        import redis
        self.connection = redis.Redis(host=host, port=port)

    def exists(self, key):
        return bool(self.connection.exists(key))

    def get(self, key):
        return self.connection.get(key)

    def set(self, key, obj):
        self.connection.set(key, obj)

    def list(self):
        cursor, keys = 0, []
        while True:
            cursor, batch = self.connection.scan(cursor=cursor, match="*")
            keys.extend(k.decode("utf-8") for k in batch)
            if cursor == 0:
                return keys


def CreateConnector(url: str) -> RemoteConnector:
    m = re.match(r"(.*)://(.*):(\d+)", url)
    if m is None:
        raise ValueError(f"Invalid remote url {url}")
    kind, host, port = m.group(1), m.group(2), int(m.group(3))
    if kind == "mem":
        return InMemoryConnector(host)
    if kind == "redis":
        return RedisConnector(host, port)
    raise ValueError(f"Invalid remote url {url} -- Unknown connector type {kind}")
