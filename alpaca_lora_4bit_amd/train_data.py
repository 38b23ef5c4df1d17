"""Dataset readers of the LoRA finetune script, with the class and method names of the reference's
src/alpaca_lora_4bit/train_data.py (`finetune.py:109-124` picks one by `--ds_type` and calls
`prepare_data(thd=..., use_eos_token=...)`, then hands `train_data` / `val_data` to the trainer).

Sample construction follows the reference:
* EOS mode (`:56-75, 138-152`): tokenize `prompt + eos_token` truncated to `cutoff_len` without padding; if
  truncation cut the EOS off and there is room, append its id (mask 1).
* padded mode (`:76-87, 153-164`): tokenize to `cutoff_len + 1` with `padding="max_length"` and drop the last
  position.
* plain text (`:107-127`): one sample per non-empty line (all files of a directory, `\\u3000` -> space there),
  optionally merged into blocks longer than `thd` characters (`:91-105`; a last block that stays at or below the
  threshold is dropped).
* Alpaca records (`:166-191`) use the instruction / input / response template; an `input` *key* is enough for the
  input section to appear, empty or not.
* GPT4All records (`:254-330`): prompt (at most half the window), newline, response without BOS, EOS when it fits;
  labels are -100 over prompt, newline and padding.
"""
import os
from abc import ABC, abstractmethod
from typing import Any, Dict

import torch

_SPLIT_SEED = 42          # train/validation split seed of the reference (train_data.py:171,235,310)


def _load_json(path):
    from datasets import load_dataset
    return load_dataset("json", data_files=path)


def _tokenize_prompt(tokenizer, prompt: str, cutoff_len: int, use_eos_token: bool) -> Dict[str, Any]:
    """The two sample shapes shared by the line, Alpaca and BlueMoon readers."""
    if not use_eos_token:
        padded = tokenizer(prompt, truncation=True, max_length=cutoff_len + 1, padding="max_length")
        return {"input_ids": padded["input_ids"][:-1], "attention_mask": padded["attention_mask"][:-1]}
    enc = tokenizer(prompt + tokenizer.eos_token, truncation=True, max_length=cutoff_len, padding=False)
    ids = enc["input_ids"]
    if ids[-1] != tokenizer.eos_token_id and len(ids) < cutoff_len:
        ids.append(tokenizer.eos_token_id)
        enc["attention_mask"].append(1)
    return enc


class ATrainData(ABC):
    """Common state: `train_data` / `val_data` are filled by `prepare_data`."""

    @abstractmethod
    def __init__(self, dataset: str, val_set_size, tokenizer, cutoff_len: int) -> None:
        self.tokenizer = tokenizer
        self.dataset = dataset
        self.val_set_size = val_set_size
        self.cutoff_len = cutoff_len
        self.train_data = None
        self.val_data = None

    @abstractmethod
    def tokenize(self, prompt: str) -> Dict[str, Any]:
        """One prompt string -> token dict."""

    @abstractmethod
    def prepare_data(self) -> None:
        """Read `self.dataset` and fill `train_data` (and `val_data`)."""


class _PromptRecords(ATrainData):
    """JSON records turned into one prompt string each (Alpaca, BlueMoon)."""

    def __init__(self, dataset: str, val_set_size, tokenizer, cutoff_len) -> None:
        super().__init__(dataset, val_set_size, tokenizer, cutoff_len)

    def tokenize(self, prompt: str, use_eos_token=True, **kwargs) -> Dict[str, Any]:
        return _tokenize_prompt(self.tokenizer, prompt, self.cutoff_len, use_eos_token)

    def generate_and_tokenize_prompt(self, data_point, **kwargs):
        return self.tokenize(self.generate_prompt(data_point, **kwargs), **kwargs)

    def prepare_data(self, use_eos_token=True, **kwargs) -> None:
        def encode(split):
            return split.shuffle().map(lambda rec: self.generate_and_tokenize_prompt(rec, use_eos_token=use_eos_token))

        records = _load_json(self.dataset)["train"]
        if self.val_set_size > 0:
            parts = records.train_test_split(test_size=self.val_set_size, shuffle=True, seed=_SPLIT_SEED)
            self.train_data, self.val_data = encode(parts["train"]), encode(parts["test"])
        else:
            self.train_data, self.val_data = encode(records), None


class TrainSAD(_PromptRecords):
    """Stanford-Alpaca-like records: instruction, optional input, output."""

    def generate_prompt(self, data_point, **kwargs):
        sections = ["Below is an instruction that describes a task, paired with an input that provides further "
                    "context. Write a response that appropriately completes the request.",
                    f"### Instruction:\n{data_point['instruction']}"]
        if "input" in data_point:
            sections.append(f"### Input:\n{data_point['input']}")
        sections.append(f"### Response:\n{data_point['output']}")
        return "\n\n".join(sections)


class TrainBlueMoon(_PromptRecords):
    """Prompt / response records."""

    def generate_prompt(self, data_point, **kwargs):
        return f"prompt:\n{data_point['prompt']}\nresponse:"      # the reference's format string has three slots (:243-248)


class TrainTxt(ATrainData):
    """Plain text, one sample per line or per merged block; the validation size is not used."""

    def __init__(self, dataset: str, val_set_size, tokenizer, cutoff_len):
        super().__init__(dataset, val_set_size, tokenizer, cutoff_len)
        self.exceed_count = 0                      # samples that fill the whole window

    def tokenize(self, prompt: str, use_eos_token=True, **kwargs) -> Dict[str, Any]:
        enc = _tokenize_prompt(self.tokenizer, prompt, self.cutoff_len, use_eos_token)
        sample = {"input_ids": enc["input_ids"], "attention_mask": enc["attention_mask"]}
        if sum(sample["attention_mask"]) >= self.cutoff_len:
            self.exceed_count += 1
        return sample

    @classmethod
    def format_new_rows(cls, rows, thd=128):
        blocks, block = [], ""
        for row in rows:
            block = row if not block else block + "\n" + row
            if len(block) > thd:
                blocks.append(block)
                block = ""
        return blocks

    def _read_rows(self):
        if os.path.isdir(self.dataset):
            rows = []
            for name in os.listdir(self.dataset):
                with open(os.path.join(self.dataset, name), "r", encoding="utf8") as fh:
                    text = fh.read().replace("\r\n", "\n").replace("　", " ")
                rows.extend(line for line in text.split("\n") if line != "")
            return rows
        with open(self.dataset, "r", encoding="utf8") as fh:
            text = fh.read().replace("\r\n", "\n")
        return [line for line in text.split("\n") if line != ""]

    def prepare_data(self, thd=-1, use_eos_token=True, **kwargs):
        from datasets import Dataset
        rows = self._read_rows()
        if thd != -1:
            rows = self.format_new_rows(rows, thd=thd)
        data = Dataset.from_dict({"input": rows})
        data = data.shuffle().map(lambda rec: self.tokenize(rec["input"], use_eos_token=use_eos_token))
        print("Train Data: {:.2f}%".format(self.exceed_count / len(data) * 100), "outliers")
        self.train_data = data


class TrainGPT4All(ATrainData):
    """Prompt / response records tokenized in batches into fixed-length rows with labels."""

    def __init__(self, dataset: str, val_set_size, tokenizer, cutoff_len) -> None:
        super().__init__(dataset, val_set_size, tokenizer, cutoff_len)

    def tokenize(self, prompt: str, use_eos_token=True, **kwargs) -> Dict[str, Any]:
        pass                                       # unused: rows are built by tokenize_inputs

    def tokenize_inputs(self, examples):
        tok, window = self.tokenizer, self.cutoff_len
        count = len(examples["prompt"])
        input_ids = torch.full((count, window), tok.pad_token_id)
        newline = tok("\n", return_tensors="pt")["input_ids"][0, 1:]          # without BOS
        labels, masks = [], []
        for i in range(count):
            head = tok(examples["prompt"][i], truncation=True, max_length=window // 2,
                       return_tensors="pt")["input_ids"].squeeze()
            if head.dim() == 0:
                head = head.unsqueeze(0)
            body_at = len(head) + len(newline)
            # the response loses its BOS and gains an EOS, hence the + 1
            room = window - len(head) - len(newline) + 1
            body = tok(examples["response"][i], truncation=True, max_length=room,
                       return_tensors="pt")["input_ids"].squeeze()[1:]
            row = input_ids[i]
            row[:len(head)] = head
            row[len(head):body_at] = newline
            row[body_at:body_at + len(body)] = body
            if body_at + len(body) < window:       # a truncated response gets no EOS
                row[body_at + len(body)] = tok.eos_token_id
            lab = row.clone()
            lab[:body_at] = -100
            lab[lab == tok.pad_token_id] = -100
            labels.append(lab)
            masks.append(row.ne(tok.pad_token_id).int())
        return {"labels": torch.stack(labels), "attention_mask": torch.stack(masks), "input_ids": input_ids}

    def prepare_data(self, **kwargs) -> None:
        def encode(split):
            return split.map(self.tokenize_inputs, batched=True, remove_columns=["source", "prompt"]).with_format("torch")

        records = _load_json(self.dataset)["train"]
        self.val_data = None
        if self.val_set_size > 0:
            parts = records.train_test_split(test_size=self.val_set_size, shuffle=True, seed=_SPLIT_SEED)
            records = parts["train"]
            self.val_data = encode(parts["test"])
        self.train_data = encode(records)
