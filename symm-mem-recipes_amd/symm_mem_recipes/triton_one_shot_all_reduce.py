"""Import-path alias: code written against the reference's module name
(symm_mem_recipes/triton_one_shot_all_reduce.py) finds the HIP implementation here.
Nothing in this package uses Triton."""
from .one_shot_all_reduce import *  # noqa: F401,F403
from .one_shot_all_reduce import main  # noqa: F401

if __name__ == "__main__":
    main()
