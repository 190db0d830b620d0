"""odla_hip: an ODLA runtime platform for one AMD Instinct MI355X (gfx950).

The product is ``libodla_hip.so`` (built from ``csrc/``); ``odla`` is the ctypes
host side that drives it through the ODLA C ABI; ``models``, ``models_yolo`` and
``models_bert`` hold the graph descriptions of the benchmark configurations.

The directory name is not a Python identifier; load the package with
``importlib`` under the name ``halo_amd`` (see ``load()`` in the repository's
``__graft_entry__.py``).
"""
from . import odla  # noqa: F401
from . import models  # noqa: F401
from . import models_bert  # noqa: F401
from . import models_yolo  # noqa: F401
from . import models_streaming  # noqa: F401
from . import calibration  # noqa: F401
from . import weights  # noqa: F401
