"""Import-path alias: code written against the reference's module name
(symm_mem_recipes/triton_barrier.py) finds the HIP implementation here.
Nothing in this package uses Triton."""
from .barrier import *  # noqa: F401,F403
from .barrier import main  # noqa: F401

if __name__ == "__main__":
    main()
