"""Import alias: ``import prime_rl_amd`` loads the package that lives in ``prime-rl_amd/``."""

import importlib
import sys

_pkg = importlib.import_module("prime-rl_amd")
for _name, _mod in list(sys.modules.items()):
    if _name == "prime-rl_amd" or _name.startswith("prime-rl_amd."):
        sys.modules["prime_rl_amd" + _name[len("prime-rl_amd"):]] = _mod
sys.modules[__name__] = _pkg
