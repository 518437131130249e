from . import creation
from . import masking
from . import nested
