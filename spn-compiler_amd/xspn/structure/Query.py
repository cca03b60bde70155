"""Query descriptions: ErrorKind, ErrorModel, Query, JointProbability.

Same constructors, defaults and accessors as the reference's xspn/xspn/structure/Query.py:13-79.
"""
from enum import IntEnum

from .Model import SPNModel  # noqa: F401


class ErrorKind(IntEnum):
    ABSOLUTE = 1
    RELATIVE = 2


class ErrorModel:
    def __init__(self, kind=ErrorKind.RELATIVE, error=0.02):
        self.kind = kind
        self.error = error


class Query:
    def __init__(self, batchSize, errorModel):
        self.batchSize = batchSize
        self.errorModel = errorModel


class JointProbability(Query):
    def __init__(self, model, batchSize=1, supportMarginal=False, rootError=ErrorModel(ErrorKind.ABSOLUTE, 0.02)):
        Query.__init__(self, batchSize, rootError)
        self.graph = model
        self.marginal = supportMarginal

    def models(self):
        return [self.graph]

    def supportsMarginal(self):
        return self.marginal
