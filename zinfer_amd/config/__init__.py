from .registry import (ArchitectureEntry, TextHooks, entry_for, load_config, read_config_json,
                       register_architecture, registered_architectures,
                       unregister_architecture)
from .specs import (GatedExpertSpec, LayerNormSpec, MoeSpec, SandwichNormBlockSpec,
                    TiedKeyValueAttentionSpec)
from .specs import (DenseMlpSpec, LatentAttentionSpec, LeadingRotarySpec, MaskedGqaAttentionSpec,
                    PostNormBlockSpec)
from .specs import (GatedLinearAttentionSpec, ParallelBlockSpec, PlainExpertSpec,
                    SinusoidalPositionSpec, TokenShiftRecurrenceSpec)
from .specs import (GqaAttentionSpec, ModelSpec, NoPositionSpec, PreNormBlockSpec, RmsNormSpec,
                    RotaryHalfSplitSpec, ScheduleEntry, SwiGluSpec)
from .qwen3 import Qwen3Config
from .fezupel import FezupelConfig
from .lodenex import LodenexConfig
from .nupovik import NupovikConfig
from .specs import GatedDeltaRuleSpec, ParallelMixerSpec, StreamBlockSpec
from .kugisun import KugisunConfig
