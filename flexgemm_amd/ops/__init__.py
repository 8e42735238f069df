from . import serialize, spconv, utils
