"""Counterpart of the reference's ``demo.py`` (:23-103) on the MI355X path: same call order --
model adapter -> ``CacheEngine(max_ctx, lm)`` -> ``add_schema(read_file(xml, [formatter]), max_tokens)`` -> ``Prompt`` ->
``process`` (with the adapter's ``use_full_position_ids``) -> ``GenerationEngine.generate`` -- run once with the prompt
cache and once with ``no_cache=True``, printing the two timed intervals of each (gather, first forward).

    python demo.py                                   # llama2-7b shape, random weights, synthetic game-like schema
    python demo.py --model falcon --schema my.xml --prompt-file my_prompt.xml
    python demo.py --model /path/to/hf/checkpoint    # real weights + tokenizer when a directory is available
    python demo.py --model kazolorn                  # the Kazolorn design (random weights), or a directory that holds one:
                                                     # plain generation, single and batched (no prompt modules for this design)
    python demo.py --model dibizen                   # the Dibizen design (lightning / attention / mamba1 layers), likewise
    python demo.py --model fivesun                   # the Fivesun design (attention / latent attention / mlstm layers), likewise
    python demo.py --model bepepel                   # the Bepepel design (gla / parallel attention + state-space layers), likewise

There is no network on the build / bench machines, so without a checkpoint directory the adapters use seeded random
weights at the named shape and the deterministic stand-in tokenizer: the text is noise, the timings are real.
"""
import argparse
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "prompt-cache_amd"))

from promptcache_amd import CacheEngine, GenerationEngine, GenerationParameters, Prompt, read_file, synth  # noqa: E402
from promptcache_amd.model import Bepepel, CodeLlama, Dibizen, Falcon, Fivesun, Kazolorn, Llama2, Mpt, load_language_model  # noqa: E402
from promptcache_amd.model.config import BepepelShape, DibizenShape, FivesunShape, KazolornShape  # noqa: E402

ADAPTERS = {"llama": (Llama2, "llama2-7b"), "codellama": (CodeLlama, "codellama-7b"), "falcon": (Falcon, "falcon-7b"),
            "mpt": (Mpt, "mpt-7b")}


def kazolorn_demo(lm, a):
    """Generation without prompt modules: one request through GenerationEngine, then a few through the batch scheduler."""
    import time
    from promptcache_amd import BatchEngine
    text = open(a.prompt_file).read() if a.prompt_file else "The quick brown fox jumps over the lazy dog. " * 8
    ids = lm.encode(text) or [1]
    params = GenerationParameters(temperature=0.0, max_new_tokens=a.max_new_tokens, stop_token_ids=[])
    last = None
    for last in GenerationEngine(lm).generate(ids, list(range(len(ids))), params):
        pass
    print(f"single : {len(ids):5d} prompt tokens | first forward {last.elapsed_time:8.3f} ms | "
          f"{a.max_new_tokens} tokens in {last.response_time:8.2f} ms")
    prompts = [ids, ids[: max(1, len(ids) // 3)], ids[: max(1, len(ids) // 2)] + ids[:5]]
    t0 = time.perf_counter()
    out = BatchEngine(lm, max_tokens=a.max_ctx).generate(prompts, params)
    dt = time.perf_counter() - t0
    print(f"batched: {len(prompts)} requests of {[len(p) for p in prompts]} tokens | {sum(len(o) for o in out)} tokens in {dt * 1e3:8.2f} ms")
    print("Assistant:", lm.decode(out[0])[:120])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="llama", help="llama | codellama | falcon | mpt | kazolorn | dibizen | fivesun | bepepel | <checkpoint directory>")
    ap.add_argument("--schema", help="PML schema file (default: a synthetic game-like schema, 7 modules)")
    ap.add_argument("--prompt-file", help="PML prompt file referencing the schema")
    ap.add_argument("--max-ctx", type=int, default=5000)
    ap.add_argument("--max-tokens", type=int, default=800)
    ap.add_argument("--max-new-tokens", type=int, default=32)
    a = ap.parse_args()

    if os.path.isdir(a.model):
        lm = load_language_model(a.model)              # the adapter class follows the directory's config.json
    elif a.model == "kazolorn":
        lm = Kazolorn(shape=KazolornShape.uniform(32000, 1024, 4, 8, 2, 128, 256, 4096, experts=8, top=2, expert_ff=1024),
                      random_init=True)
    elif a.model == "dibizen":
        lm = Dibizen(shape=DibizenShape.uniform(32000, 1024, ["lightning", "attention", "mamba1", "attention"], 8, 2, 128, 8, 2, 1024,
                                                identity=2, groups=2, groups_keep=1, max_positions=max(a.max_ctx, 4096)),
                     random_init=True)
    elif a.model == "fivesun":
        lm = Fivesun(shape=FivesunShape.uniform(32000, 1024, ["attention", "latent_attention", "attention", "mlstm"], 8, 2, 128, 2048,
                                                chunk=1024, window=512, kv_rank=192, rot_dim=64), random_init=True)
    elif a.model == "bepepel":
        lm = Bepepel(shape=BepepelShape.uniform(32000, 1024, ["gla", "parallel", "gla", "gla"], 8, 2, 128, experts=8, top=2, expert_ff=512,
                                                window=512, keep_first=4), random_init=True)
    else:
        cls, shape = ADAPTERS[a.model]
        lm = cls(shape, random_init=True)
    if isinstance(lm, (Kazolorn, Dibizen, Fivesun, Bepepel)):
        kazolorn_demo(lm, a)
        return
    preproc = [lm.get_formatter()]
    cache_engine = CacheEngine(a.max_ctx, lm)
    gen_engine = GenerationEngine(lm)
    if a.schema:
        cache_engine.add_schema(read_file(a.schema, preproc), max_tokens=a.max_tokens)
        prompt_text = open(a.prompt_file).read()
    else:
        schema_text, prompt_text = synth.flat_docs("code-generation-game", 30, (306, 76, 800, 800, 800, 800, 800), 12)
        cache_engine.add_schema(lm.get_formatter()(schema_text), max_tokens=a.max_tokens)
    params = GenerationParameters(temperature=1.0, repetition_penalty=1.0, top_p=0.95, top_k=-1,
                                  max_new_tokens=a.max_new_tokens, stop_token_ids=lm.stop_token_ids, stop_str=lm.stop_str)
    prompt = Prompt(prompt_text, preproc)
    for no_cache in (False, True, False):       # the first pass also warms the hipGraph / allocator
        token_ids, position_ids, cache_time, cache = cache_engine.process(
            prompt, no_cache=no_cache, return_full_position_ids=lm.use_full_position_ids)
        last = None
        for last in gen_engine.generate(token_ids, position_ids, params, cache, stream_interval=2,
                                        use_full_position_ids=lm.use_full_position_ids):
            pass
        staged = 0 if cache is None else cache[0][0].shape[1]
        print(f"{'no_cache' if no_cache else 'cached  '}: staged {staged:5d} + new {len(token_ids):5d} tokens | "
              f"gather {cache_time:7.3f} ms | first forward {last.elapsed_time:8.3f} ms | "
              f"TTFT {cache_time + last.elapsed_time:8.3f} ms | {a.max_new_tokens} tokens in {last.response_time:8.2f} ms")
    print("Assistant:", (last.new_text[:120] + " ...") if last else "")


if __name__ == "__main__":
    main()
