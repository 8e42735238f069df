from . import spconv, utils
