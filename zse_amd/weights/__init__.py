from .loader import CheckpointWeights, RandomWeights, WeightError, check_entries, check_folder
from .random_init import write_random_model
