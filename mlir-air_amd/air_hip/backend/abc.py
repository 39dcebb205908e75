"""Backend interface, same contract as the reference's AirBackend
(python/air/backend/abc.py:23-61): compile(module) -> artifact,
load(artifact) -> invoker; errors raise AirBackendError."""

import abc


class AirBackend(abc.ABC):
    @abc.abstractmethod
    def compile(self, module):
        """Turn a module description into an artifact that `load` understands."""

    @abc.abstractmethod
    def load(self, artifact):
        """Return a callable invoker(*ndarrays) -> tuple of ndarrays."""


class AirBackendError(Exception):
    def __init__(self, message):
        super().__init__(message)
