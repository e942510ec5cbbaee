"""Text in and out: the chat template against the two renderings that the reference's own
test holds, the byte tokenizer, and streaming."""
import json

import llama_cu_amd
from llama_cu_amd import text

# llama.cu/src/model/chat_template.rs:134-135: the two templates of the reference's test
TAIDE = ("{% if messages[0]['role'] == 'system' %}{% set loop_messages = messages[1:] %}{% set system_message = "
         "'<<SYS>>\n' + messages[0]['content'] + '\n<</SYS>>\n\n' %}{% else %}{% set loop_messages = messages %}"
         "{% set system_message = '' %}{% endif %}{% for message in loop_messages %}{% if loop.index0 == 0 %}"
         "{% set content = system_message + message['content'] %}{% else %}{% set content = message['content'] %}"
         "{% endif %}{% if message['role'] == 'user' %}{{ bos_token + '[INST] ' + content + ' [/INST]'}}"
         "{% elif message['role'] == 'assistant' %}{{ ' '  + content + ' ' + eos_token }}{% endif %}{% endfor %}"
         "{% if add_generation_prompt %}{{ '<|im_start|>assistant\n' }}{% endif %}")
MINICPM = ("{% for message in messages %}{% if message['role'] == 'user' %}{{'<用户>' + message['content'].strip() + "
           "'<AI>'}}{% else %}{{message['content'].strip()}}{% endif %}{% endfor %}")


def test_the_reference_s_two_renderings():
    """llama.cu/src/model/chat_template.rs:137-149."""
    msg = [text.user("Hello, who are you?")]
    assert text.ChatTemplate(TAIDE, "<s>", "</s>").render(msg, True) == \
        "<s>[INST] Hello, who are you? [/INST]<|im_start|>assistant\n"
    assert text.ChatTemplate(MINICPM, "<s>", "</s>").render(msg, True) == "<用户>Hello, who are you?<AI>"


def test_system_message_and_turns():
    t = text.ChatTemplate(TAIDE, "<s>", "</s>")
    out = t.render([{"role": "system", "content": "Be brief."}, text.user("Hi"), {"role": "assistant", "content": "Yo"},
                    text.user("Bye")], False)
    assert out == "<s>[INST] <<SYS>>\nBe brief.\n<</SYS>>\n\nHi [/INST] Yo </s><s>[INST] Bye [/INST]"


def test_template_of_a_model_folder(tmp_path):
    (tmp_path / "tokenizer_config.json").write_text(json.dumps(
        {"chat_template": MINICPM, "bos_token": {"content": "<s>"}, "eos_token": "</s>"}))
    assert text.load_chat_template(str(tmp_path)).render([text.user(" x ")]) == "<用户>x<AI>"
    assert "user: x" in text.load_chat_template(str(tmp_path / "none")).render([text.user("x")])


def test_byte_tokenizer_and_streaming():
    tok = text.load_tokenizer("/nonexistent", 256)
    ids = tok.encode("héllo ✓")
    assert all(0 <= i < 256 for i in ids) and tok.decode(ids) == "héllo ✓"
    dec = text.StreamDecoder(tok)
    pieces = [dec.push(i) for i in ids]
    assert "".join(pieces) == "héllo ✓"
    assert "" in pieces                                 # a character's first bytes are held back
    import pytest
    with pytest.raises(ValueError):
        text.ByteTokenizer(100)


def test_a_tokenizer_file_is_read_and_round_trips(tmp_path):
    """A small word-level ``tokenizer.json`` made with the ``tokenizers`` package: a folder that
    holds one gets it, and text goes to ids and back."""
    import pytest
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    vocab = {"[UNK]": 0, "hello": 1, "world": 2, "once": 3, "upon": 4, "a": 5, "time": 6, ",": 7}
    tk = Tokenizer(models.WordLevel(vocab, unk_token="[UNK]"))
    tk.pre_tokenizer = pre_tokenizers.Whitespace()
    tk.decoder = decoders.Fuse()
    tk.save(str(tmp_path / "tokenizer.json"))
    tok = text.load_tokenizer(str(tmp_path), 8)
    assert isinstance(tok, text.FileTokenizer)
    ids = tok.encode("once upon a time, hello")
    assert ids == [3, 4, 5, 6, 7, 1]
    assert tok.encode("hello zebra") == [1, 0]                    # what the file does not know
    assert tok.decode([1, 2]).replace(" ", "") == "helloworld"
    dec = text.StreamDecoder(tok)
    assert "".join(dec.push(i) for i in [3, 4]).replace(" ", "") == "onceupon"
