"""Host-side callers of the path (CPU): command line and settings object, dataset readers, activation checkpointing.
The expectations are the reference's documented behaviour (src/alpaca_lora_4bit/arg_parser.py,
Finetune4bConfig.py, train_data.py, gradient_checkpointing.py), checked on hand-made inputs."""
import json
import os

import numpy as np
import pytest
import torch


# ------------------------------------------------------------------ arg_parser / Finetune4bConfig
def test_command_line_defaults_match_the_reference():
    from alpaca_lora_4bit_amd.arg_parser import parse_commandline
    got = parse_commandline([])
    want = dict(dataset="./dataset.json", ds_type="alpaca", lora_out_dir="alpaca_lora", lora_apply_dir=None,
                resume_checkpoint=None, llama_q4_config_dir="./llama-13b-4bit/", llama_q4_model="./llama-13b-4bit.pt",
                mbatch_size=1, batch_size=2, epochs=3, lr=2e-4, cutoff_len=256, lora_r=8, lora_alpha=16,
                lora_dropout=0.05, grad_chckpt=False, grad_chckpt_ratio=1, val_set_size=0.2, warmup_steps=50,
                save_steps=50, save_total_limit=3, logging_steps=10, checkpoint=False, skip=False, verbose=False,
                txt_row_thd=-1, use_eos_token=1, groupsize=-1, v1=False, local_rank=0, flash_attention=False,
                xformers=False, backend="cuda")
    assert got == want


def test_get_config_derives_what_the_reference_derives(monkeypatch):
    from alpaca_lora_4bit_amd.arg_parser import get_config
    monkeypatch.delenv("WORLD_SIZE", raising=False)
    monkeypatch.delenv("LOCAL_RANK", raising=False)
    cfg = get_config(["data.txt", "--ds_type", "txt", "--batch_size", "32", "--mbatch_size", "4", "--grad_chckpt",
                      "--lora_dropout", "0.1", "--val_set_size", "200", "--use_eos_token", "0", "-c", "--groupsize",
                      "128", "--backend", "triton", "--lora_r", "16"])
    assert cfg.dataset == "data.txt" and cfg.ds_type == "txt" and cfg.checkpoint and cfg.groupsize == 128
    assert cfg.gradient_accumulation_steps == 8
    assert cfg.gradient_checkpointing and cfg.lora_dropout == 0            # dropout is switched off with checkpointing
    assert cfg.val_set_size == 200 and isinstance(cfg.val_set_size, int)     # > 1: a row count
    assert cfg.use_eos_token is False and cfg.backend == "triton" and cfg.lora_r == 16
    assert cfg.world_size == 1 and not cfg.ddp and cfg.device_map == "auto" and cfg.local_rank == 0
    text = str(cfg)
    assert "gradient_accumulation_steps=8" in text and "dataset='data.txt'" in text and "self." not in text

    frac = get_config(["--val_set_size", "0.1"])
    assert frac.val_set_size == 0.1 and isinstance(frac.val_set_size, float) and frac.lora_dropout == 0.05

    monkeypatch.setenv("WORLD_SIZE", "4")
    monkeypatch.setenv("LOCAL_RANK", "3")
    ddp = get_config(["--batch_size", "32", "--mbatch_size", "2"])
    assert ddp.ddp and ddp.device_map == {"": 3} and ddp.gradient_accumulation_steps == 4   # 32 // 2 // 4


def test_unknown_dataset_type_is_rejected():
    from alpaca_lora_4bit_amd.arg_parser import parse_commandline
    with pytest.raises(SystemExit):
        parse_commandline(["--ds_type", "parquet"])


# ------------------------------------------------------------------ train_data
class ToyTokenizer:
    """One token per whitespace-separated word; ids: pad 0, bos 1, eos 2, words from 3.  Mimics the call
    signature of a Hugging Face tokenizer as far as the readers use it."""
    pad_token_id, bos_token_id, eos_token_id = 0, 1, 2
    eos_token = "</s>"

    def __init__(self):
        self.vocab = {}

    def _ids(self, text):
        ids = [self.bos_token_id]
        for word in text.replace(self.eos_token, " " + self.eos_token + " ").split():
            ids.append(self.eos_token_id if word == self.eos_token else self.vocab.setdefault(word, 3 + len(self.vocab)))
        return ids

    def __call__(self, text, truncation=False, max_length=None, padding=False, return_tensors=None):
        ids = self._ids(text)
        if truncation and max_length is not None:
            ids = ids[:max_length]
        mask = [1] * len(ids)
        if padding == "max_length":
            ids, mask = ids + [self.pad_token_id] * (max_length - len(ids)), mask + [0] * (max_length - len(mask))
        if return_tensors == "pt":
            return {"input_ids": torch.tensor([ids]), "attention_mask": torch.tensor([mask])}
        return {"input_ids": ids, "attention_mask": mask}


def test_eos_and_padded_sample_shapes():
    from alpaca_lora_4bit_amd.train_data import TrainSAD, TrainTxt
    tok = ToyTokenizer()
    sad = TrainSAD("unused.json", 0, tok, cutoff_len=6)
    short = sad.tokenize("a b c")
    assert short["input_ids"] == [1, 3, 4, 5, 2] and short["attention_mask"] == [1] * 5     # bos a b c eos
    cut = sad.tokenize("a b c d e f g")                   # truncated to the window: the EOS is cut off and there is no room
    assert len(cut["input_ids"]) == 6 and cut["input_ids"][-1] != tok.eos_token_id
    padded = sad.tokenize("a b", use_eos_token=False)     # window + 1 padded, last position dropped
    assert padded["input_ids"] == [1, 3, 4, 0, 0, 0] and padded["attention_mask"] == [1, 1, 1, 0, 0, 0]

    txt = TrainTxt("unused.txt", 0, tok, cutoff_len=4)
    assert set(txt.tokenize("a b c d e")) == {"input_ids", "attention_mask"} and txt.exceed_count == 1
    txt.tokenize("a")
    assert txt.exceed_count == 1                          # only samples that fill the window count


def test_alpaca_prompt_template():
    from alpaca_lora_4bit_amd.train_data import TrainBlueMoon, TrainSAD
    sad = TrainSAD("unused.json", 0, ToyTokenizer(), 32)
    with_input = sad.generate_prompt({"instruction": "Add.", "input": "1 2", "output": "3"})
    assert with_input == ("Below is an instruction that describes a task, paired with an input that provides further "
                          "context. Write a response that appropriately completes the request.\n\n"
                          "### Instruction:\nAdd.\n\n### Input:\n1 2\n\n### Response:\n3")
    assert "### Input:\n\n\n" in sad.generate_prompt({"instruction": "x", "input": "", "output": "y"})   # key present
    assert "### Input" not in sad.generate_prompt({"instruction": "x", "output": "y"})
    moon = TrainBlueMoon("unused.json", 0, ToyTokenizer(), 32)
    assert moon.generate_prompt({"prompt": "p", "response": "r"}) == "prompt:\np\nresponse:"


def test_text_rows_are_merged_past_the_threshold_and_the_short_tail_is_dropped():
    from alpaca_lora_4bit_amd.train_data import TrainTxt
    rows = ["aaaa", "bbbb", "cc", "dddddddddd", "e"]
    assert TrainTxt.format_new_rows(rows, thd=8) == ["aaaa\nbbbb", "cc\ndddddddddd"]       # "e" never exceeds 8
    assert TrainTxt.format_new_rows(rows, thd=3) == ["aaaa", "bbbb", "cc\ndddddddddd"]


def test_text_reader_on_a_file_and_a_directory(tmp_path):
    from alpaca_lora_4bit_amd.train_data import TrainTxt
    one = tmp_path / "one.txt"
    one.write_text("first line\r\n\r\nsecond line\nthird\n", encoding="utf8")
    data = TrainTxt(str(one), 0, ToyTokenizer(), cutoff_len=8)
    data.prepare_data()
    assert len(data.train_data) == 3 and data.val_data is None
    assert sorted(len(r["input_ids"]) for r in data.train_data) == [3, 4, 4]      # bos + words + eos

    folder = tmp_path / "many"
    folder.mkdir()
    (folder / "a.txt").write_text("x　y\nz\n", encoding="utf8")
    (folder / "b.txt").write_text("w\n", encoding="utf8")
    both = TrainTxt(str(folder), 0, ToyTokenizer(), cutoff_len=8)
    both.prepare_data(thd=-1, use_eos_token=False)
    assert len(both.train_data) == 3
    assert all(len(r["input_ids"]) == 8 for r in both.train_data)                 # padded mode: fixed length
    assert sorted(sum(r["attention_mask"]) for r in both.train_data) == [2, 2, 3]  # ideographic space became a blank


def test_alpaca_reader_splits_and_tokenizes(tmp_path):
    from alpaca_lora_4bit_amd.train_data import TrainSAD
    path = tmp_path / "alpaca.json"
    records = [{"instruction": f"do {i}", "input": "", "output": f"done {i}"} for i in range(10)]
    path.write_text(json.dumps(records))
    data = TrainSAD(str(path), 0.2, ToyTokenizer(), cutoff_len=64)
    data.prepare_data(use_eos_token=True)
    assert len(data.train_data) == 8 and len(data.val_data) == 2
    row = data.train_data[0]
    assert row["input_ids"][0] == 1 and row["input_ids"][-1] == 2 and len(row["input_ids"]) == len(row["attention_mask"])
    no_val = TrainSAD(str(path), 0, ToyTokenizer(), cutoff_len=64)
    no_val.prepare_data()
    assert len(no_val.train_data) == 10 and no_val.val_data is None


def test_gpt4all_rows_and_labels():
    from alpaca_lora_4bit_amd.train_data import TrainGPT4All
    tok = ToyTokenizer()
    data = TrainGPT4All("unused.json", 0, tok, cutoff_len=10)
    out = data.tokenize_inputs({"prompt": ["p q", "a b c d e f g"], "response": ["r s t", "u v w x y z"]})
    nl = []                                              # the toy tokenizer maps "\n" to no token at all
    ids, lab, mask = out["input_ids"], out["labels"], out["attention_mask"]
    assert ids.shape == lab.shape == mask.shape == (2, 10)
    # row 0: bos p q | r s t | eos | padding
    p, q, r, s, t = (tok.vocab[w] for w in "pqrst")
    assert ids[0].tolist() == [1, p, q] + nl + [r, s, t, 2, 0, 0, 0]
    assert lab[0].tolist() == [-100] * 3 + [r, s, t, 2, -100, -100, -100]
    assert mask[0].tolist() == [1] * 7 + [0] * 3
    # row 1: the prompt is cut to half the window (bos + 4 words), the response fills the rest, no room for an EOS
    a, b, c, d = (tok.vocab[w] for w in "abcd")
    resp = [tok.vocab[w] for w in "uvwxy"]
    assert ids[1].tolist() == [1, a, b, c, d] + resp and 2 not in ids[1].tolist()
    assert lab[1].tolist() == [-100] * 5 + resp


# ------------------------------------------------------------------ gradient_checkpointing
def test_checkpoint_locations():
    from alpaca_lora_4bit_amd.gradient_checkpointing import checkpoint_locations
    assert checkpoint_locations(4, 1).tolist() == [0, 1, 2, 3]
    assert checkpoint_locations(4, 2.0).tolist() == [0, 1, 2, 3]          # outside (0, 1): every block
    assert checkpoint_locations(32, 0.25).tolist() == [0, 4, 9, 13, 18, 22, 27, 31]     # 8 blocks, first to last
    assert checkpoint_locations(10, 0.5).tolist() == [0, 2, 4, 7, 9]


def test_checkpointed_blocks_give_the_same_gradients():
    from transformers import LlamaConfig, LlamaForCausalLM
    from alpaca_lora_4bit_amd.gradient_checkpointing import NewForward, VarWrapper, apply_gradient_checkpointing
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=97, hidden_size=32, intermediate_size=64, num_hidden_layers=4, num_attention_heads=4,
                      num_key_value_heads=4, max_position_embeddings=64)
    model = LlamaForCausalLM(cfg).float().train()
    model.config.use_cache = False
    ids = torch.randint(0, 97, (2, 12))
    watched = ["model.layers.0.self_attn.q_proj.weight", "model.layers.3.mlp.down_proj.weight", "lm_head.weight"]

    def grads():
        model.zero_grad()
        model(input_ids=ids, labels=ids, use_cache=False).loss.backward()
        named = dict(model.named_parameters())
        return [named[n].grad.clone() for n in watched], named["model.embed_tokens.weight"].grad

    plain, emb_grad = grads()
    assert emb_grad is not None
    patched, wrapper = apply_gradient_checkpointing(model, checkpoint_ratio=0.5)
    assert len(patched) == 2 and all(isinstance(p, NewForward) for p in patched) and isinstance(wrapper, VarWrapper)
    assert [hasattr(l, "old_forward_for_cp") for l in model.model.layers] == [True, False, False, True]
    calls = {"n": 0}
    inner = model.model.layers[0].old_forward_for_cp

    def counting(*a, **k):
        calls["n"] += 1
        return inner(*a, **k)

    model.model.layers[0].old_forward_for_cp = counting
    again, emb_grad2 = grads()
    assert calls["n"] == 2                                # forward + recomputation in backward
    for g0, g1 in zip(plain, again):
        assert torch.allclose(g0, g1, rtol=1e-5, atol=1e-7)
    assert emb_grad2 is None or float(emb_grad2.abs().max()) == 0.0     # the graph is cut after the embedding
    model.eval()
    calls["n"] = 0
    with torch.no_grad():
        model(input_ids=ids, use_cache=False)
    assert calls["n"] == 1                                # no checkpointing outside training mode


def test_token_picker_of_the_graph_decode():
    """inference._token_picker: argmax without sampling settings; with the reference's settings (inference.py:33-44)
    the draw comes from the top-k set after repetition penalty and temperature, through transformers' processors."""
    import torch
    from alpaca_lora_4bit_amd import inference
    logits = torch.tensor([[0.1, 2.0, 5.0, 4.9, -1.0, 3.0]])
    ids = torch.tensor([[2, 2]])
    assert inference._token_picker(None)(ids, logits).tolist() == [[2]]
    torch.manual_seed(0)
    pick = inference._token_picker({"repetition_penalty": 1.1, "temperature": 0.9, "top_k": 2, "top_p": 0.95})
    draws = {int(pick(ids, logits.clone())) for _ in range(200)}
    assert draws <= {2, 3} and draws == {2, 3}            # top-2 after the penalty on token 2: {3, 2}
    # a huge penalty on the already generated token 2 leaves token 3 as the only survivor of top-p
    pick = inference._token_picker({"repetition_penalty": 50.0, "temperature": 0.1, "top_k": 2, "top_p": 0.5})
    assert {int(pick(ids, logits.clone())) for _ in range(50)} == {3}
