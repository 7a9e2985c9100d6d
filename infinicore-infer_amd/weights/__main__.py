"""python -m infinicore_infer_amd.weights --config config.json --seed S --out DIR: the random-weights mode."""
import sys

from .random_init import main

sys.exit(main())
