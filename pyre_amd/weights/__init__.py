from pyre_amd.weights.loader import WeightsError, adopt_state, checkpoint_index, load_weights
from pyre_amd.weights.random_init import model_tensor_specs, random_state, write_random_model

__all__ = ["WeightsError", "adopt_state", "checkpoint_index", "load_weights", "model_tensor_specs",
           "random_state", "write_random_model"]
