"""Drop-in import name: `import expert_specialization` / `from expert_specialization.ops import ...`
work as with the reference package (expert_specialization/__init__.py:1-3); everything is provided by
expert_specialization_moe_amd."""
from expert_specialization_moe_amd import *  # noqa: F401,F403
from expert_specialization_moe_amd import _native as _C  # noqa: F401  (the reference exposes `_C`)
