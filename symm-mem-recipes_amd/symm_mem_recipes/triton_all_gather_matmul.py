"""Import-path alias: code written against the reference's module name
(symm_mem_recipes/triton_all_gather_matmul.py) finds the HIP implementation here.
Nothing in this package uses Triton."""
from .all_gather_matmul import *  # noqa: F401,F403
from .all_gather_matmul import main  # noqa: F401

if __name__ == "__main__":
    main()
