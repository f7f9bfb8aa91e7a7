from .generation import GenerationSession, ModelConfig, RaggedGenerationSession, SamplingConfig
from .kv_cache_manager import GenerationSequence, KVCacheManager, StateSlotManager
from .scheduler import RaggedScheduler, Request
from .session import Session, TensorInfo

__all__ = ['ModelConfig', 'GenerationSession', 'RaggedGenerationSession', 'RaggedScheduler', 'Request', 'StateSlotManager', 'GenerationSequence', 'KVCacheManager', 'SamplingConfig', 'Session',
           'TensorInfo']
