"""A Python entry point shaped like the reference's torch class ``gpt_ops.OptOp``
(src/csrc/pybinding.cc:53-62, src/csrc/model/gpt/opt/optop.cc:9-36,
src/csrc/model/gpt/gptop_base.cc:40-75): the caller owns the K/V cache tensors and
the block tables and calls ``forward`` with whole prompts or single decode tokens.

    op = OptOp(vocab_size, max_position_embeddings, hidden_size, num_layers, num_heads,
               head_dim, inference_dtype, block_size, max_num_block_per_req, parallel_config)
    op.load_weight(model_dir)  |  op.init_dummy_weights()
    tokens = op.forward(input_tokens_batched, first_token_indexes, k_cache, v_cache, block_table)

``k_cache``/``v_cache``: [num_blocks, num_layers, num_heads, block_size, head_dim]
(src/csrc/model/gpt/gpt_base.h:70-72).  ``first_token_indexes[i]`` is the number of tokens
request i already has in the cache (0 for a whole prompt).  Unlike the reference, a request
may also bring a portion of a prompt with a non-zero first index.  Returns one greedy token
per request.  ``forward_logits`` returns the float logits of each request's last token."""
from __future__ import annotations

from typing import List, Sequence

import torch

from .config.hyper_param import OptHyperParam
from .engine.batch import StepItem, pack_batch
from .engine.engine import parse_dtype
from .models import build_model
from .cache.device import CacheView
from .ops import kernels as K
from .weights.random_init import file_dtype_of, random_tensors


class OptOp:
    def __init__(self, vocab_size: int, max_position_embeddings: int, hidden_size: int,
                 num_layers: int, num_heads: int, head_dim: int, inference_dtype: str,
                 block_size: int, max_num_block_per_req: int, parallel_config: Sequence[int] = (1, 0, 1, 0),
                 ffn_dim: int = 0, device: str = "cuda:0"):
        if num_heads * head_dim != hidden_size:
            raise ValueError("num_heads * head_dim must equal hidden_size")   # attention.cc:82
        pc = list(parallel_config)    # [tp_size, tp_rank, pp_size, pp_rank]
        if (len(pc) > 0 and pc[0] != 1) or (len(pc) > 2 and pc[2] != 1):
            raise ValueError("this engine runs on one GPU: tensor and pipeline sizes must be 1")
        # the reference's OptOp fixes the feed-forward width to 4 * hidden (optop.cc:28)
        self.hyper_param = OptHyperParam(
            vocab_size=vocab_size, max_position_embeddings=max_position_embeddings,
            hidden_size=hidden_size, num_hidden_layers=num_layers, num_attention_heads=num_heads,
            ffn_dim=ffn_dim or 4 * hidden_size, word_embed_proj_dim=hidden_size).validate()
        self.dtype = parse_dtype(inference_dtype)
        self.device = torch.device(device)
        self.block_size = block_size
        self.max_num_block_per_req = max_num_block_per_req
        self.model = build_model(self.hyper_param, self.dtype)

    def load_weight(self, path: str) -> None:
        self.model.load_weights(path, self.device)

    def init_dummy_weights(self, seed: int = 0) -> None:
        self.model.bind(random_tensors(self.model.tensor_specs(), seed, self.dtype, self.device,
                                       file_dtype=file_dtype_of(self.hyper_param)))

    def init_communicator(self, tp_id, pp_id) -> None:
        """Single GPU: nothing to set up (kept for callers of the reference's interface)."""

    def forward_logits(self, input_tokens_batched, first_token_indexes, k_cache, v_cache,
                       block_table) -> torch.Tensor:
        if not self.model.weights_loaded:
            raise RuntimeError("Please load the weight before inference.")   # gptop_base.cc:47-49
        hp = self.hyper_param
        L, nh, hd, bs = hp.num_hidden_layers, hp.num_attention_heads, hp.head_dim, self.block_size
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dim() != 5 or tuple(c.shape[1:]) != (L, nh, bs, hd) or c.dtype != self.dtype:
                raise ValueError(f"{name} must be [num_blocks, {L}, {nh}, {bs}, {hd}] of {self.dtype}")
        items = [StepItem(slot=i, start=int(first), tokens=[int(t) for t in toks],
                          want=[len(toks) - 1], pages={0: [int(b) for b in bt]})
                 for i, (toks, first, bt) in enumerate(zip(input_tokens_batched, first_token_indexes,
                                                           block_table))]
        ctx = pack_batch(items, [0], self.max_num_block_per_req, bs, self.device,
                         vocab_size=hp.vocab_size, max_positions=hp.max_position_embeddings,
                         planners=self.model.step_planners())
        views = {l: CacheView(l, 0, k=k_cache[:, l], v=v_cache[:, l]) for l in range(L)}
        return self.model.forward(ctx, views)

    def forward(self, input_tokens_batched, first_token_indexes, k_cache, v_cache, block_table) -> List[int]:
        if len(input_tokens_batched) == 0:
            return []                                                         # gptop_base.cc:52-54
        logits = self.forward_logits(input_tokens_batched, first_token_indexes, k_cache, v_cache,
                                     block_table)
        return K.sample(logits).cpu().tolist()
