"""Engine-level configuration and the request-facing records, with the reference's names.

EngineConfig  : /root/reference/src/utils/config.rs:421-492, Python face xinfer.pyi:47-140
SamplingParams: /root/reference/src/utils/config.rs:797-832, xinfer.pyi:142-151
GenerationConfig / GenerationOutput / Message: xinfer.pyi:30-45,153-157
Options of the reference that belong to parts not built here (quantisation, several GPUs,
prefix cache, server, speculative decoding) are absent rather than accepted and ignored.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import List, Optional, Tuple, Union


class DType(Enum):
    """The reference's names (xinfer.pyi:8-11).  Half precision (F16) is not built: the engine
    refuses it when it is made."""
    F16 = "f16"
    BF16 = "bf16"
    F32 = "f32"


@dataclass
class GenerationConfig:
    """Sampling defaults of a model (generation_config.json in the reference,
    /root/reference/src/utils/mod.rs:1868-1889)."""
    temperature: Optional[float] = None
    top_p: Optional[float] = None
    top_k: Optional[int] = None
    frequency_penalty: Optional[float] = None
    presence_penalty: Optional[float] = None
    eos_token_id: Tuple[int, ...] = ()     # one id or a list in the file; joined with config.json's (config.rs:360-375)


@dataclass
class SamplingParams:
    temperature: Optional[float] = None
    max_tokens: Optional[int] = None
    ignore_eos: bool = False
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    session_id: Optional[str] = None
    frequency_penalty: Optional[float] = None
    presence_penalty: Optional[float] = None
    seed: Optional[int] = None          # per-request seed; default: the engine's seed and the request id
    # Generation ends when the new token completes one of these (config.rs:807-809): texts, tokenised
    # at admission, and/or token id sequences.  The completing token is not appended (as with EOS);
    # the earlier tokens of a longer stop sequence stay in the output, as in the reference.
    stop_sequences: Optional[List[str]] = None
    stop_token_ids: Optional[List[List[int]]] = None


@dataclass
class Message:
    role: str
    content: str
    num_images: int = 0         # the reference's field (xinfer.pyi:151-155); text only here, so it must stay 0


@dataclass
class GenerationOutput:
    seq_id: int
    prompt_length: int
    prompt_start_time: int      # milliseconds since the epoch, as in the reference
    decode_start_time: int
    decode_finish_time: int
    decoded_length: int
    decode_output: str
    token_ids: List[int] = field(default_factory=list)     # the generated token ids
    finish_reason: str = ""                                 # "eos", "stop", "length", "max_model_len"


@dataclass(frozen=True)
class StreamItem:
    """An item of an `EngineStream` (xinfer.pyi:160-180).  datatype / data:
    "TOKEN" / the token's text; "TOKEN_ID" / its id; "DONE" / (prompt_start_time,
    decode_start_time, decode_finish_time, decoded_length); "COMPLETION" / (prompt_start_time,
    decode_start_time, decode_finish_time, token ids), the one item of a request that is not
    streamed; "ERROR" / a message."""
    datatype: str
    data: object


@dataclass
class EngineConfig:
    model_id: Optional[str] = None          # a local model folder (there is no hub download here)
    weight_path: Optional[str] = None       # the same, under the reference's legacy name
    max_num_seqs: int = 32                  # most requests live at a time
    max_model_len: Optional[int] = None     # default: the positions the model can encode (max_position_embeddings, more under YaRN)
    max_tokens: Optional[int] = None        # default per request: 16384, clipped to max_model_len
    generation_cfg: Optional[GenerationConfig] = None
    seed: Optional[int] = None
    kv_fraction: Optional[float] = None     # share of free GPU memory given to the cache (0.6)
    prefill_chunk_size: int = 8192          # most prompt tokens of one request in a step (any >= 1)
    disable_cuda_graph: bool = False        # the reference's name; here it disables HIP graphs
    yarn_scaling_factor: Optional[float] = None   # YaRN over the model's own length, in place of its rope_scaling
    # --- this engine's own ---
    page_size: int = 64                     # tokens per cache page (the reference fixes 64)
    num_pages: Union[int, List[int], None] = None   # pages of every cache group, or one count per group; default: from kv_fraction
    max_num_batched_tokens: Optional[int] = None   # token budget of a step; default: chunk size
    device: str = "cuda:0"
    # launch a step before the tokens of the step before it have been read on the host (they
    # reach it on the device); False: every step's tokens are read before the next is planned
    run_ahead: bool = True

    def model_dir(self) -> str:
        if self.model_id and self.weight_path:
            raise ValueError("Use either model_id (--m) or weight_path (--w), not both.")
        d = self.model_id or self.weight_path
        if not d:
            raise ValueError("Must provide model_id or weight_path!")
        return d
