"""The asynchronous engine: coroutines that stream at the same time are batched together and
each gets the tokens the plain implementation generates; leaving a stream early takes the
request out; a prompt that cannot be served fails its caller alone."""

import asyncio

import pytest

import plain_qwen3
from helpers import TINY, random_tokens
from qwen3_from_scratch_amd.engine import LLMEngine


def _plain_greedy(folder, prompts, n):
    cfg, w = plain_qwen3.read_model_folder(folder)
    return [plain_qwen3.greedy_generate(cfg, w, p, n) for p in prompts]


async def _collect(engine, prompt, n, **kw):
    chunks = []
    async for chunk in engine.generate_stream(prompt, max_new_tokens=n, ignore_eos=True, temperature=0.0, **kw):
        chunks.append(chunk)
    return chunks


def _scenario(folder, name, device, dtype, want_exact):
    vocab = TINY[name]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (9, 40, 3, 25)]
    want = _plain_greedy(folder, prompts, 10)
    engine = LLMEngine(path=folder, dtype=dtype, device=device, block_size=TINY[name]["page_size"], num_blocks=40,
                       max_num_seqs=3, max_num_tokens=32, chunked_prefill_size=16)
    manager = None

    async def main():
        await engine.warmup()
        # four callers at once (one more than the engine runs at a time), the last arriving a little later
        async def late():
            await asyncio.sleep(0.01)
            return await _collect(engine, prompts[3], 10)
        results = await asyncio.gather(_collect(engine, prompts[0], 10), _collect(engine, prompts[1], 10),
                                       _collect(engine, prompts[2], 10), late())
        for prompt, chunks, tokens in zip(prompts, results, want):
            got = [c.token_id for c in chunks]
            if want_exact:
                assert got == tokens
            else:
                assert len(got) == 10 and got[0] == tokens[0]
            assert [c.metrics.token_count for c in chunks] == list(range(1, 11))
            assert chunks[0].metrics.tps == 0.0 and chunks[-1].metrics.total_elapsed >= chunks[0].metrics.ttft > 0
            assert chunks[0].prompt_tokens == len(prompt) and len({c.req_id for c in chunks}) == 1
        # a caller that leaves after two tokens: its request is taken out
        seen = 0
        async for _ in engine.generate_stream(prompts[1], max_new_tokens=30, ignore_eos=True, temperature=0.0):
            seen += 1
            if seen == 2:
                break
        # a prompt longer than the cache fails its own caller; the engine goes on
        with pytest.raises(ValueError):
            await _collect(engine, [1] * 5000, 4)
        with pytest.raises(ValueError):
            await _collect(engine, [{"role": "user", "content": "hello"}], 4)      # no tokenizer in the folder
        again = await _collect(engine, prompts[0], 10)
        assert [c.token_id for c in again][:1] == want[0][:1]

    try:
        engine.wait_ready()
        manager = engine.engine.runner.manager
        asyncio.run(main())
    finally:
        engine.close()
    assert not engine.thread.is_alive()
    manager.audit()
    assert manager.num_free() == 40 and not manager.live()


def test_concurrent_streams_on_the_host(cpu_ops, model_folders):
    _scenario(model_folders["B"], "B", "cpu", "float32", True)


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("E", "bfloat16")])
def test_concurrent_streams_on_the_gpu(model_folders, name, dtype):
    _scenario(model_folders[name], name, "cuda", dtype, dtype == "float32")


def test_an_engine_that_cannot_start_says_so(tmp_path):
    engine = LLMEngine(path=str(tmp_path / "nothing_here"), device="cpu")
    with pytest.raises(RuntimeError):
        engine.wait_ready()
    engine.close()
