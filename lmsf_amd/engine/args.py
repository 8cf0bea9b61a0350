"""Engine arguments with the reference's option names and meanings
(core/src/common/config.rs:9-87), as a dataclass and as command-line flags.

Options of the reference that have no meaning here are still accepted, so that its command lines
run: --swap-space, --max-paddings, --threads, --chat-template are parsed and unused (as --threads and
--chat-template are in the reference); --log-dir and --alsologtostderr switch on the engine's log; --tp, --pp must be 1
and --quantization must be absent, or the engine refuses to start.
"""
import argparse
import dataclasses
from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineArgs:
    model: str = ""
    dtype: Optional[str] = None                    # default: config.json's torch_dtype
    max_model_len: Optional[int] = None            # default: config.json's max_position_embeddings
    block_size: int = 16
    seed: int = 0
    gpu_memory_utilization: float = 0.9
    max_num_batched_tokens: Optional[int] = None   # default: max(max_model_len, 2048)
    max_num_seqs: int = 256
    max_paddings: int = 256                        # unused: batches have no padding
    swap_space: int = 4                            # unused: preemption recomputes
    quantization: Optional[str] = None
    chat_template: Optional[str] = ""
    pipeline_parallel_size: int = 1
    tensor_parallel_size: int = 1
    threads: int = 4
    log_dir: Optional[str] = None
    alsologtostderr: bool = False
    # beyond the reference
    load_format: str = "auto"                      # "auto": safetensors of the folder; "random": random weights
    prefill_chunk_size: Optional[int] = None
    num_gpu_blocks_override: Optional[int] = None
    enforce_eager: bool = False                    # True: never capture decode steps as HIP graphs
    run_ahead: bool = True                         # False: never launch a step before the tokens of the one before are read
    tune_products: bool = False                    # True: at load, the BLAS library's candidates race for the products of a full step
    keep_float32_weights: bool = False             # True: matrices stored in 32 bits are not cast to a bfloat16 run's type
    skip_tokenizer_init: bool = False              # True: work on token ids even if the folder has a tokenizer.json
    device: str = "cuda:0"

    def verify(self) -> None:
        if self.quantization:
            raise ValueError("--quantization %s: quantized weights are not supported" % self.quantization)
        if self.pipeline_parallel_size != 1 or self.tensor_parallel_size != 1:
            raise ValueError("--pp and --tp must be 1: this engine runs on one GPU")
        if self.gpu_memory_utilization > 1.0 or self.gpu_memory_utilization <= 0.0:
            # core/src/common/config.rs:245-250
            raise ValueError("GPU memory utilization must be in (0, 1]. Got %r." % self.gpu_memory_utilization)
        if self.load_format not in ("auto", "random"):
            raise ValueError("--load-format must be auto or random")

    @staticmethod
    def add_cli_args(parser: argparse.ArgumentParser) -> argparse.ArgumentParser:
        a = parser.add_argument
        a("--model", required=True, help="path of the huggingface model folder to use")
        a("--dtype", default=None, choices=["float32", "bfloat16", "float16", "half", "auto"],
          help="the datatype to use for model (float16 runs as bfloat16)")
        a("--max-model-len", type=int, default=None,
          help="model context length. If unspecified, will be automatically derived from the model")
        a("--block-size", type=int, default=16, help="token block size")
        a("--seed", type=int, default=0, help="random seed")
        a("--gpu-memory-utilization", type=float, default=0.9,
          help="the percentage of GPU memory to be used for the model executor")
        a("--max-num-batched-tokens", type=int, default=None, help="maximum number of batched tokens per iteration")
        a("--max-num-seqs", type=int, default=256, help="maximum number of sequences per iteration")
        a("--max-paddings", type=int, default=256, help="maximum number of paddings in a batch (unused)")
        a("--swap-space", type=int, default=4, help="CPU swap space size (GiB) per GPU (unused)")
        a("--quantization", default=None, help="specify quantize method (not supported)")
        a("--chat-template", default="", help="chat template config file (unused)")
        a("--pp", dest="pipeline_parallel_size", type=int, default=1, help="number of pipeline stages (1)")
        a("--tp", dest="tensor_parallel_size", type=int, default=1, help="number of tensor parallel replicas (1)")
        a("--threads", type=int, default=4, help="(unused)")
        a("--log-dir", default=None, help="log dir (lmsf.log in it, a new file every day)")
        a("--alsologtostderr", action="store_true", help="print log into stderr")
        a("--load-format", default="auto", choices=["auto", "random"],
          help="auto: the folder's safetensors; random: random weights for the folder's config.json")
        a("--prefill-chunk-size", type=int, default=None, help="longest portion of a prompt in one step")
        a("--num-gpu-blocks-override", type=int, default=None, help="pages of the cache instead of sizing from memory")
        a("--enforce-eager", action="store_true", help="run decode steps kernel by kernel instead of as HIP graphs")
        a("--no-run-ahead", dest="run_ahead", action="store_false",
          help="launch a step only after the tokens of the step before it have been read")
        a("--skip-tokenizer-init", action="store_true", help="do not load the folder's tokenizer.json")
        a("--tune-products", action="store_true",
          help="at load, time the BLAS library's candidate algorithms for the matrix products of a step of "
               "--max-num-batched-tokens tokens (and of --prefill-chunk-size) on the model's own weights and keep the "
               "fastest of each")
        a("--keep-float32-weights", action="store_true",
          help="with --dtype bfloat16, leave matrices that the checkpoint stores in 32 bits as they are (their "
               "products then run in float32 arithmetic, at twice the memory) instead of casting them at load")
        a("--device", default="cuda:0")
        return parser

    @classmethod
    def from_cli_args(cls, ns: argparse.Namespace) -> "EngineArgs":
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in vars(ns).items() if k in names})
