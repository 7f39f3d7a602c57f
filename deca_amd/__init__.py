"""DeCA operator auto-tuner, MI355X (gfx950) build.

Public surface (same names as the reference's `src/` tree): `Solver`,
`RuntimeMod`, `Tuner`, `cost_model.CostModel`, `operators`, `kernels`, `arch`.
Importing the package touches neither torch nor the GPU.
"""

__all__ = ["arch", "kernels", "operators", "cost_model", "driver", "utils"]
