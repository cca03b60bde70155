"""SPNModel: an SPN graph plus the type of its input features and a name.

Same constructor and attributes as the reference's xspn/xspn/structure/Model.py:13-33.
"""
import numpy as np


class SPNModel:
    def __init__(self, rootNode, featureValueType=np.dtype(np.float64).name, modelName=None):
        self.root = rootNode
        self.featureType = featureValueType
        self.name = modelName
