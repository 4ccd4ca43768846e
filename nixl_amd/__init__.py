"""MI355X-native implementation of NIXL's descriptor-transfer and expert-parallel
dispatch/combine hot path.  Native code lives in ``nixl_amd/csrc`` and is loaded through
ctypes (``nixl_amd._lib``); torch is used only to own device memory and streams."""
from .agent import (NIXL_INIT_AGENT, NixlError, nixl_agent, nixl_agent_config)  # noqa: F401

__all__ = ["nixl_agent", "nixl_agent_config", "NixlError", "NIXL_INIT_AGENT"]
