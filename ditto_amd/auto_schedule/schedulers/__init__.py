from . import chimera_integrate
