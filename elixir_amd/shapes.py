"""Parameter lists (name, shape) of the model families the optimizer-step workloads are quoted on.
Only shapes: the step is element-wise, so a workload is fully described by its tensor sizes, their
order (which fixes the packing into chunks) and which tensors are exempt from weight decay.
"""
from typing import List, Tuple

NamedShape = Tuple[str, Tuple[int, ...]]


def gpt2_shapes(n_layer: int = 12, hidden: int = 768, vocab: int = 50257, n_pos: int = 1024) -> List[NamedShape]:
    """GPT-2 (Conv1D layout); defaults are GPT-2 small: 148 tensors, 124,439,808 elements."""
    out: List[NamedShape] = [('wte.weight', (vocab, hidden)), ('wpe.weight', (n_pos, hidden))]
    for i in range(n_layer):
        p = f'h.{i}.'
        out += [
            (p + 'ln_1.weight', (hidden, )),
            (p + 'ln_1.bias', (hidden, )),
            (p + 'attn.c_attn.weight', (hidden, 3 * hidden)),
            (p + 'attn.c_attn.bias', (3 * hidden, )),
            (p + 'attn.c_proj.weight', (hidden, hidden)),
            (p + 'attn.c_proj.bias', (hidden, )),
            (p + 'ln_2.weight', (hidden, )),
            (p + 'ln_2.bias', (hidden, )),
            (p + 'mlp.c_fc.weight', (hidden, 4 * hidden)),
            (p + 'mlp.c_fc.bias', (4 * hidden, )),
            (p + 'mlp.c_proj.weight', (4 * hidden, hidden)),
            (p + 'mlp.c_proj.bias', (hidden, )),
        ]
    out += [('ln_f.weight', (hidden, )), ('ln_f.bias', (hidden, ))]
    return out


def opt_shapes(n_layer: int = 24, hidden: int = 2048, ffn: int = 8192, vocab: int = 50272,
               n_pos: int = 2050) -> List[NamedShape]:
    """OPT decoder; defaults are OPT-1.3B: 388 tensors, 1,315,758,080 elements (tied lm_head)."""
    out: List[NamedShape] = [('embed_tokens.weight', (vocab, hidden)), ('embed_positions.weight', (n_pos, hidden))]
    for i in range(n_layer):
        p = f'layers.{i}.'
        for proj in ('k_proj', 'v_proj', 'q_proj', 'out_proj'):
            out += [(p + f'self_attn.{proj}.weight', (hidden, hidden)), (p + f'self_attn.{proj}.bias', (hidden, ))]
        out += [
            (p + 'self_attn_layer_norm.weight', (hidden, )),
            (p + 'self_attn_layer_norm.bias', (hidden, )),
            (p + 'fc1.weight', (ffn, hidden)),
            (p + 'fc1.bias', (ffn, )),
            (p + 'fc2.weight', (hidden, ffn)),
            (p + 'fc2.bias', (hidden, )),
            (p + 'final_layer_norm.weight', (hidden, )),
            (p + 'final_layer_norm.bias', (hidden, )),
        ]
    out += [('final_layer_norm.weight', (hidden, )), ('final_layer_norm.bias', (hidden, ))]
    return out


def llama_shapes(n_layer: int = 32, hidden: int = 4096, ffn: int = 11008, vocab: int = 32000) -> List[NamedShape]:
    """LLaMA; defaults are LLaMA-7B: 291 tensors, 6,738,415,616 elements."""
    out: List[NamedShape] = [('embed_tokens.weight', (vocab, hidden))]
    for i in range(n_layer):
        p = f'layers.{i}.'
        out += [
            (p + 'self_attn.q_proj.weight', (hidden, hidden)),
            (p + 'self_attn.k_proj.weight', (hidden, hidden)),
            (p + 'self_attn.v_proj.weight', (hidden, hidden)),
            (p + 'self_attn.o_proj.weight', (hidden, hidden)),
            (p + 'mlp.gate_proj.weight', (ffn, hidden)),
            (p + 'mlp.up_proj.weight', (ffn, hidden)),
            (p + 'mlp.down_proj.weight', (hidden, ffn)),
            (p + 'input_layernorm.weight', (hidden, )),
            (p + 'post_attention_layernorm.weight', (hidden, )),
        ]
    out += [('norm.weight', (hidden, )), ('lm_head.weight', (vocab, hidden))]
    return out


def numel(shape: Tuple[int, ...]) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


def no_decay(name: str, shape: Tuple[int, ...]) -> bool:
    """The usual exemption: biases and normalisation weights (every 1-D tensor) take no decay."""
    return len(shape) == 1
