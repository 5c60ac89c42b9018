from .batch import StepBatch, pack_step
from .context import StepContext
from .generate import (GenerationOptions, GenerationResult, LoopDetector, SequenceTrack, generate,
                       plan_batches)
from .model import (CausalLM, build_block, load_model, model_from_config, random_model,
                    write_random_model_dir)
from .step import Engine, StepError
