"""The text path on the GPU: ``LLM.generate`` from texts and conversations, the chat program fed a
dialogue on its standard input, and the generate program with every kind of record and prompt,
all on a tiny model whose vocabulary is the fixture tokenizer's."""

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from .helpers import TINY_A, make_folder, read_folder
from .test_gpu_generate import plain_greedy
from .text_fixture import EOT, ID, SPECIALS, WORDS, write_tokenizer

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
# (untied: with tied embeddings a random model repeats its last prompt token, a special one, and says nothing)
CONFIG = dict(TINY_A, vocab_size=len(WORDS) + len(SPECIALS), tie_word_embeddings=False)


@pytest.fixture(scope="module")
def talker(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("text") / "m", CONFIG, seed=8, dtype=torch.float32, sharpen=True)
    write_tokenizer(folder)
    cfg, weights = read_folder(folder)
    return folder, cfg, weights


def test_generate_from_conversations_and_texts(talker):
    from torchllms_amd.inference import LLM
    from torchllms_amd.messages.templates import LLAMA3_INSTRUCT, tokenize_conversation

    folder, cfg, weights = talker
    llm = LLM(str(folder), template_config="llama3_instruct", precision="float32", max_len=96, max_bsz=2, page_size=8)
    assert llm.eos_ids == [128009]  # the template's stop ids win (reference: llm.py:188-189)
    conversations = [
        [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hello world"}],
        [{"role": "user", "content": "how are you <|eot_id|>"}],
    ]
    ids = [tokenize_conversation(c, llm.tokenizer, LLAMA3_INSTRUCT) for c in conversations]
    assert ids[1].count(EOT) == 1  # the envelope's; the one spelt out in the content is plain text
    by_text = llm.generate(conversations=conversations, max_new_tokens=7)
    by_ids = llm.generate(prompt_token_ids=ids, max_new_tokens=7)
    for text, tok, prompt in zip(by_text, by_ids, ids):
        assert text.token_ids == tok.token_ids == plain_greedy(weights, cfg, prompt, 7)
        assert text.text == llm.tokenizer.decode(text.token_ids) == tok.text and len(text.text.split()) >= 3
    # plain prompts: encoded without added special tokens
    prompts = ["hello world again", "fine"]
    got = llm.generate(prompts=prompts, max_new_tokens=5)
    want = llm.generate(prompt_token_ids=[[ID["hello"], ID["world"], ID["again"]], [ID["fine"]]], max_new_tokens=5)
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    # an explicit stop id ends a turn, and the stop token stays out of the text
    first = by_text[0].token_ids[2]
    r = llm.generate(conversations=conversations[:1], max_new_tokens=7, stop_token_ids=[first])[0]
    assert r.token_ids == by_text[0].token_ids[: by_text[0].token_ids.index(first) + 1] and r.stop_reason == first
    with pytest.raises(ValueError, match="exactly one"):
        llm.generate(prompts=prompts, conversations=conversations)
    bare = LLM(str(folder), precision="float32", max_len=64, max_bsz=1)
    with pytest.raises(ValueError, match="template_config"):
        bare.generate(conversations=conversations)


def _assistant_lines(stdout: str):
    return [line.split("[assistant]: \033[0m", 1)[1] for line in stdout.splitlines() if "[assistant]: " in line]


def test_chat_program_with_reset(talker):
    """[system], a user turn, a second turn that sees the first answer, ``!!reset``, an empty system
    line, a user turn, then the end of input: three answers, each the model's for the conversation so far."""
    from torchllms_amd.inference import LLM

    folder, _, _ = talker
    llm = LLM(str(folder), template_config="llama3_instruct", precision="float32", max_len=128, max_bsz=1)
    say = lambda conv: llm.generate(conversations=[conv], max_new_tokens=6)[0].text
    first = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hello world"}]
    a1 = say(first)
    second = first + [{"role": "assistant", "content": a1}, {"role": "user", "content": "how are you"}]
    a2 = say(second)
    a3 = say([{"role": "user", "content": "thanks"}])
    cmd = [sys.executable, "-m", "torchllms_amd.inference.chat", "--ckpt_paths", str(folder), "--template_config", "llama3_instruct",
           "--precision", "float32", "--max_new_tokens", "6", "--max_len", "128"]
    proc = subprocess.run(cmd, input="be brief\nhello world\nhow are you\n!!reset\n\nthanks\n", capture_output=True, text=True,
                          cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert all(len(a.split()) >= 3 for a in (a1, a2, a3)) and len({a1, a2, a3}) == 3  # answers with words in them, all different
    assert _assistant_lines(proc.stdout) == [a1, a2, a3]
    # prompts: two [system] (start and reset), five [user] (three turns, the reset, and the one that met the end of input)
    assert proc.stdout.count("[system]: ") == 2 and proc.stdout.count("[user]: ") == 5
    # the dashed spellings name the same options
    cmd = [sys.executable, "-m", "torchllms_amd.inference.chat", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "6",
           "--max-model-len", "128"]
    proc = subprocess.run(cmd, input="\nthanks\n", capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0 and _assistant_lines(proc.stdout) == [a3]


def test_generate_program_with_messages_prompts_and_single_prompts(talker, tmp_path):
    from torchllms_amd.inference import LLM

    folder, cfg, weights = talker
    llm = LLM(str(folder), template_config="llama3_instruct", precision="float32", max_len=128, max_bsz=2)
    provider = json.dumps({"ckpt_paths": str(folder), "precision": "float32", "max_len": 128, "template_config": "llama3_instruct"})
    base = [sys.executable, "-m", "torchllms_amd.inference.generate"]

    def run(args, **kw):
        proc = subprocess.run(base + args, capture_output=True, text=True, cwd=ROOT, timeout=300, **kw)
        assert proc.returncode == 0, proc.stderr[-2000:]
        return proc.stdout

    # records with messages: each conversation grows by the assistant's answer
    conversations = [[{"role": "user", "content": "hello world"}], [{"role": "system", "content": "be brief"}, {"role": "user", "content": "how are you"}]]
    inp, out = tmp_path / "m.jsonl", tmp_path / "m_out.jsonl"
    inp.write_text("".join(json.dumps({"messages": c, "tag": i}) + "\n" for i, c in enumerate(conversations)))
    run(["--input_path", str(inp), "--output_path", str(out), "--provider_kwargs", provider, "--generate_kwargs", '{"max_new_tokens": 5}'])
    want = llm.generate(conversations=conversations, max_new_tokens=5)
    recs = [json.loads(l) for l in out.read_text().splitlines()]
    assert [r["tag"] for r in recs] == [0, 1]
    for rec, conv, res in zip(recs, conversations, want):
        assert rec["messages"] == conv + [{"role": "assistant", "content": res.text}]
    # records with prompts: the answer is the completion
    inp.write_text(json.dumps({"prompt": "hello world again"}) + "\n" + json.dumps({"prompt": "fine thanks"}) + "\n")
    run(["--input_path", str(inp), "--output_path", str(out), "--provider_kwargs", provider, "--generate_kwargs", '{"max_new_tokens": 5}'])
    want = llm.generate(prompts=["hello world again", "fine thanks"], max_new_tokens=5)
    assert [json.loads(l)["completion"] for l in out.read_text().splitlines()] == [r.text for r in want]
    # one prompt on the command line, as text and as ids
    text = run(["--model", str(folder), "--dtype", "float32", "--prompt", "hello world again", "--max-new-tokens", "5"])
    assert text.strip().splitlines()[-1] == want[0].text
    prompt = [ID["how"], ID["are"], ID["you"]]
    ids = run(["--model", str(folder), "--dtype", "float32", "--prompt-ids", *map(str, prompt), "--max-new-tokens", "5"])
    assert [int(t) for t in ids.strip().splitlines()[-1].split()] == plain_greedy(weights, cfg, prompt, 5)
    # bad combinations are refused by the parser
    proc = subprocess.run(base + ["--model", str(folder), "--prompt", "x", "--prompt-ids", "1"], capture_output=True, text=True, cwd=ROOT)
    assert proc.returncode == 2 and "exactly one" in proc.stderr


def test_random_weights_from_the_command_line(tmp_path):
    """``--random-weights --seed N``: the folder holds config.json (and a tokenizer) only; the weights
    are those that the random-weights mode writes for that seed."""
    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.weights import write_model_folder

    cfg_obj = LlamaConfig.from_dict(CONFIG)
    written = write_model_folder(tmp_path / "written", cfg_obj, seed=4, dtype=torch.float32)
    cfg, weights = read_folder(written)
    bare = tmp_path / "bare"
    bare.mkdir()
    (bare / "config.json").write_text((written / "config.json").read_text())
    write_tokenizer(bare)
    prompt = [ID["hello"], ID["world"]]
    cmd = [sys.executable, "-m", "torchllms_amd.inference.generate", "--model", str(bare), "--random-weights", "--seed", "4",
           "--dtype", "float32", "--prompt-ids", *map(str, prompt), "--max-new-tokens", "6"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.strip().splitlines()[-1].split()] == plain_greedy(weights, cfg, prompt, 6)
    chat = [sys.executable, "-m", "torchllms_amd.inference.chat", "--model", str(bare), "--random-weights", "--seed", "4", "--dtype", "float32",
            "--max-new-tokens", "4", "--max-model-len", "64"]
    proc = subprocess.run(chat, input="\nhello world\n", capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0 and len(_assistant_lines(proc.stdout)) == 1, proc.stderr[-2000:]
