"""MuiModule -- muillm/modules/module.py:6-32: base class of every replacement layer with
the finalize_init()/finalize_deinit() protocol run by init_engine."""
import torch.nn as nn

from ..engineconfig import MuiEngineConfig


class MuiModule(nn.Module):
    def __init__(self, engine_config: MuiEngineConfig = None, **kargs) -> None:
        if engine_config is None:
            # a cooperative super().__init__() from a class with several bases: the real
            # initialisation call with an engine config follows
            return None
        nn.Module.__init__(self, **kargs)
        self.engine_config = engine_config

    def __del__(self):
        try:
            self.finalize_deinit()
        except Exception:
            pass

    def finalize_init(self) -> None:
        """Called post-order once all layers are replaced and on their device."""

    def finalize_deinit(self) -> None:
        """Called on destruction."""
