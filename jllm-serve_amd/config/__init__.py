"""Typed configuration: schema records, the architecture registry, the Qwen3 parser."""
from .schema import (ConfigError, GatedMlpNames, GatedMlpSpec, GqaNames, GqaSpec, LatentAttentionNames,
                     LatentAttentionSpec, LayerSpec, ModelConfig, ModelNames, NormSpec, RopeScaling, RopeSpec,
                     ScheduleEntry, TableMoeNames, TableMoeSpec, default_schedule)
from .registry import (entry_for, load_config, parse_config, register_architecture, supported,
                       unregister_architecture)
from . import qwen3 as _qwen3  # registers "qwen3"
from . import miforax as _miforax  # registers "miforax"
from . import kebepel as _kebepel  # registers "kebepel"
from . import ratasun as _ratasun  # registers "ratasun"
from . import pivipel as _pivipel  # registers "pivipel"

__all__ = ["ConfigError", "GatedMlpNames", "GatedMlpSpec", "GqaNames", "GqaSpec", "LatentAttentionNames", "LatentAttentionSpec", "TableMoeNames", "TableMoeSpec", "ModelNames", "LayerSpec", "ModelConfig", "NormSpec", "RopeScaling", "RopeSpec",
           "ScheduleEntry", "default_schedule", "entry_for", "load_config", "parse_config", "register_architecture",
           "supported", "unregister_architecture"]
