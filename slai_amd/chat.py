"""Headless chat over the C ABI: the loop of crates/slai-chat/src/cli.rs:35-164 and
crates/slai-chat/src/chat_llama2.rs:64-162 with the tokenizer, the sampler and the decode loop of libslai_hip.

    python -m slai_amd.chat MODEL.gguf [--inspect] [--greedy] [--temperature T] [--top-p P] [--seed N]

The model file is mapped, parsed and uploaded; every turn renders the conversation through the chat template
(`tokenizer.chat_template`, else a Llama-2 `[INST]` template), tokenizes it, and resumes the decode loop at the
position where the previous turn stopped.  Tokens are picked on the device (`Sampler::new(vocab, 0.7, 0.95)` like
crates/slai-chat/src/sampler.rs:107), a few at a time, so only token ids cross the bus.
"""
import argparse
import sys
import time

import numpy as np

from . import _ffi
from .runtime import Backend, Gguf, Llama2, Tokenizer

# The Llama-2 chat layout: <s>[INST] <<SYS>>\nsystem\n<</SYS>>\n\nuser [/INST] assistant </s><s>[INST] user [/INST]
DEFAULT_CHAT_TEMPLATE = (
    "{%- set ns = namespace(sys='') -%}"
    "{%- if messages and messages[0]['role'] == 'system' -%}"
    "{%- set ns.sys = '<<SYS>>\\n' ~ (messages[0]['content'] | trim) ~ '\\n<</SYS>>\\n\\n' -%}"
    "{%- set messages = messages[1:] -%}"
    "{%- endif -%}"
    "{%- for m in messages -%}"
    "{%- if m['role'] == 'user' -%}{{ bos_token }}[INST] {{ ((ns.sys if loop.first else '') ~ m['content']) | trim }} [/INST]"
    "{%- elif m['role'] == 'assistant' %} {{ m['content'] | trim }} {{ eos_token }}{%- endif -%}"
    "{%- endfor -%}"
)


class Prompt:
    """crates/slai-chat/src/prompt.rs:43-108: the conversation so far."""

    def __init__(self):
        self.entries = []

    def append_user(self, text):
        self.entries.append(("user", text))

    def append_assistant(self, text):
        self.entries.append(("assistant", text))

    def append_system(self, text):
        self.entries.append(("system", text))

    def clear(self):
        self.entries.clear()

    def messages(self):
        return [dict(role=r, content=c) for r, c in self.entries]


class ChatTemplate:
    """crates/slai-chat/src/chat_template.rs:10-39 with jinja2 in place of minijinja."""

    def __init__(self, template):
        self.template = template

    @classmethod
    def from_gguf(cls, gguf):
        try:
            return cls(gguf.meta_str("tokenizer.chat_template"))
        except Exception:
            return cls(DEFAULT_CHAT_TEMPLATE)

    def apply(self, prompt, bos, eos):
        import jinja2

        def raise_exception(msg):
            raise jinja2.TemplateError(msg)

        env = jinja2.Environment(trim_blocks=True)
        env.globals.update(bos_token=bos, eos_token=eos, add_generation_prompt=True, raise_exception=raise_exception)
        return env.from_string(self.template).render(messages=prompt.messages())


def model_type_of(gguf):
    """crates/slai-chat/src/llm.rs:38-58: the architecture name selects the variant."""
    name = gguf.meta_str("general.architecture").lower()
    if "llama" in name:
        return _ffi.MODEL_LLAMA
    if "qwen2" in name:
        return _ffi.MODEL_QWEN2
    raise ValueError("Unrecognized model")


class ChatLlm:
    """``ChatLlama2`` (chat_llama2.rs): model + tokenizer, one conversation."""

    def __init__(self, backend, gguf, kv_dtype=_ffi.KV_F16, temperature=0.7, topp=0.95, seed=0, chunk=8):
        self.model = Llama2(backend, gguf, model_type_of(gguf), kv_dtype)
        self.tokenizer = Tokenizer(gguf)
        self.template = ChatTemplate.from_gguf(gguf)
        self.temperature, self.topp, self.seed, self.chunk = temperature, topp, seed, chunk
        self.seq_len = self.model.config.seq_len

    def forward(self, prompt, start_pos, on_token=None, max_new_tokens=None):
        """chat_llama2.rs:64-162: returns (text, next_pos, n_generated, seconds).  `on_token(piece)` is called per token."""
        tk = self.tokenizer
        text = self.template.apply(prompt, tk.bos_str(), tk.eos_str())
        toks = tk.encode(text, False, False)                       # :86
        if not toks or start_pos >= len(toks):
            return "", start_pos, 0, 0.0
        fed = list(toks)                                            # token fed at each position
        out_text, pos, n_new, t0, t_start = [], start_pos, 0, None, start_pos + 1
        next_pos = start_pos                                        # position of the last reported token (cli.rs:139)
        done = False
        # the prompt up to its last token in chunks (no logits are needed there: the tokens are forced,
        # slai-chat/src/sampler.rs:100-105); the loop below then starts at the last prompt token
        if hasattr(self.model, "prefill") and len(toks) - 1 - pos >= 8:
            self.model.prefill(np.asarray(toks[pos:len(toks) - 1], np.int32), pos)
            pos = len(toks) - 1
            t_start = pos + 1
        while not done and pos < self.seq_len:
            steps = min(self.chunk if pos + 1 >= len(toks) else (len(toks) - 1 - pos) + self.chunk, self.seq_len - pos)
            ids, _ = self.model.generate_sampled(np.asarray(fed, np.int32), steps, self.temperature, self.topp, self.seed, start_pos=pos)
            for nxt in ids.tolist():
                if pos == t_start:
                    t0 = time.perf_counter()                        # :119-121: the first token is not timed
                prev = fed[pos]
                if pos + 1 >= len(toks):                            # past the prompt: a generated token (:135)
                    if nxt == tk.eos:
                        done = True
                        break
                    piece = tk.decode([nxt], prev_token=prev)       # :130
                    out_text.append(piece)
                    n_new += 1
                    next_pos = pos
                    if on_token:
                        on_token(piece)
                    if len(fed) <= pos + 1:
                        fed.append(nxt)
                    if max_new_tokens is not None and n_new >= max_new_tokens:
                        pos += 1
                        done = True
                        break
                pos += 1
        seconds = (time.perf_counter() - t0) if t0 is not None else 0.0
        return "".join(out_text), next_pos, n_new, seconds

    def close(self):
        self.tokenizer.close()
        self.model.destroy()


def inspect(gguf):
    """`gguf.print_metadata()` and `gguf.print_tensors()` (crates/slai/src/gguf.rs:681-711)."""
    for line in gguf.metadata_debug_strings():
        print(line)
    tensors = gguf.tensors()
    for name in sorted(tensors):
        print("%s -> %s" % (name, tensors[name]["dims"]))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("path")
    ap.add_argument("--inspect", action="store_true")
    ap.add_argument("--greedy", action="store_true", help="temperature 0")
    ap.add_argument("--temperature", type=float, default=0.7)
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--seed", type=int, default=int(time.time()))
    ap.add_argument("--kv", choices=["f16", "f32"], default="f16")
    args = ap.parse_args(argv)
    t = time.perf_counter()
    gguf = Gguf.open(args.path)
    print("GGUF model loaded in %.2f seconds." % (time.perf_counter() - t))
    if args.inspect:
        inspect(gguf)
    t = time.perf_counter()
    backend = Backend(0)
    llm = ChatLlm(backend, gguf, _ffi.KV_F16 if args.kv == "f16" else _ffi.KV_F32, 0.0 if args.greedy else args.temperature, args.top_p, args.seed)
    print("Uploaded model to GPU in %.2f seconds." % (time.perf_counter() - t))
    print("Starting interactive chat:")
    prompt, next_pos = Prompt(), 0
    while True:
        print("[User]")
        line = sys.stdin.readline()
        if not line:
            break
        prompt.append_user(line.rstrip())
        print("[Assistant]")
        last = [""]

        def show(piece):
            if last[0] != "\n" or piece != "\n":                   # cli.rs:133-137: no runs of empty lines
                sys.stdout.write(piece)
                sys.stdout.flush()
            last[0] = piece

        text, next_pos, n, seconds = llm.forward(prompt, next_pos, show)
        print()
        print("(%.2f tok/s) - generated %d tokens" % ((max(n - 1, 0) / seconds) if seconds > 0 else 0.0, next_pos))
        prompt.append_assistant(text)
    llm.close()
    backend.close()
    gguf.close()


if __name__ == "__main__":
    main()
