"""Chat templates and stop ids come from the model folder, never from code (CPU only)."""

import json

from rapid_llm_amd.engine.prompting import ChatPrompter, build_prompter, is_instruct, read_chat_template
from rapid_llm_amd.engine.tokenizer import load_stop_token_ids, load_tokenizer

# a template written for this test, in the dialect model folders use
TEMPLATE = (
    "{{ bos_token }}{% for m in messages %}"
    "{% if m['role'] not in ['system', 'user', 'assistant'] %}{{ raise_exception('unknown role') }}{% endif %}"
    "<{{ m['role'] }}>{{ m['content'] }}</{{ m['role'] }}>{{ eos_token if m['role'] == 'assistant' else '' }}\n"
    "{% endfor %}{% if add_generation_prompt %}<assistant>{% endif %}"
)


def _folder(tmp_path, name="tiny", model_type="qwen3", **tokenizer_config):
    folder = tmp_path / name
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps({"model_type": model_type}))
    if tokenizer_config:
        (folder / "tokenizer_config.json").write_text(json.dumps(tokenizer_config))
    return folder


def _word_tokenizer(folder, words):
    from tokenizers import Tokenizer, models, pre_tokenizers

    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token=words[0]))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(str(folder / "tokenizer.json"))


def test_the_template_is_the_folders_own(tmp_path):
    folder = _folder(tmp_path, chat_template=TEMPLATE, bos_token="<s>", eos_token={"content": "</s>"})
    prompter = build_prompter(folder)
    assert prompter.insert_prompt("hello") == "<s><user>hello</user>\n<assistant>"
    talk = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "a"},
            {"role": "assistant", "content": "b"}, {"role": "user", "content": "c"}]
    assert prompter.apply(talk) == (
        "<s><system>be brief</system>\n<user>a</user>\n<assistant>b</assistant></s>\n<user>c</user>\n<assistant>"
    )
    assert prompter.apply(talk[:2], add_generation_prompt=False).endswith("</user>\n")
    try:
        prompter.apply([{"role": "tool", "content": "x"}])
    except ValueError as exc:
        assert "unknown role" in str(exc)
    else:
        raise AssertionError("the template's own refusal was swallowed")
    # a template file beside the tokenizer wins over the entry in tokenizer_config.json
    (folder / "chat_template.jinja").write_text("{{ messages[0]['content'] }}!")
    assert build_prompter(folder).insert_prompt("hi") == "hi!"
    assert build_prompter(folder, use_template=False) is None


def test_without_a_template_prompts_go_in_as_they_are(tmp_path):
    assert build_prompter(_folder(tmp_path, "plain")) is None
    assert read_chat_template(_folder(tmp_path, "empty", eos_token="</s>")) is None
    named = _folder(tmp_path, "named", chat_template=[{"name": "tool", "template": "T"},
                                                      {"name": "default", "template": "D"}])
    assert read_chat_template(named) == "D"


def test_base_checkpoints_are_told_from_instruction_tuned_ones(tmp_path):
    """rapid_llm/utils/prompt_templates.py:76-150: the folder's name first, then the model type."""
    assert is_instruct(_folder(tmp_path, "Some-7B-Instruct", model_type="llama"))
    assert not is_instruct(_folder(tmp_path, "Some-7B", model_type="llama"))
    assert is_instruct(_folder(tmp_path, "Qwen3-8B"))
    assert not is_instruct(_folder(tmp_path, "Qwen3-8B-Base", chat_template=TEMPLATE))
    assert build_prompter(tmp_path / "Qwen3-8B-Base") is None  # a base model's template is a trap


def test_stop_ids_are_the_tokenizers_and_the_generation_configs(tmp_path):
    """rapid_llm/engine/stop_criteria.py:29-54: both sources count."""
    words = ["<unk>", "a", "b", "</s>", "<end_turn>"]
    folder = _folder(tmp_path, eos_token={"content": "</s>", "special": True})
    _word_tokenizer(folder, words)
    tokenizer = load_tokenizer(folder)
    assert load_stop_token_ids(folder, (), tokenizer) == {3}
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [4, 3]}))
    assert load_stop_token_ids(folder, (), tokenizer) == {3, 4}
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": 4}))
    assert load_stop_token_ids(folder, (1,), tokenizer) == {1, 3, 4}
    (folder / "generation_config.json").write_text("{ broken")
    assert load_stop_token_ids(folder, (), tokenizer) == {3}
    # an id written out in tokenizer_config.json, a token the vocabulary lacks, no tokenizer at all
    assert load_stop_token_ids(_folder(tmp_path, "by_id", eos_token_id=2), (), None) == {2}
    assert load_stop_token_ids(_folder(tmp_path, "unknown", eos_token="<nowhere>"), (), tokenizer) == set()
    assert load_stop_token_ids(None, (7,), None) == {7}

    class WithId:
        eos_token_id = 9

    assert load_stop_token_ids(folder, (), WithId()) == {9}


def test_whether_an_architecture_chats_by_default_is_its_registry_entrys_flag(tmp_path):
    """No architecture is named beside the prompt code: a newly registered one says itself
    whether its releases are chat models, and one that is not registered gets prompts verbatim."""
    from rapid_llm_amd.config import register_architecture, unregister_architecture

    class ToyConfig:
        @classmethod
        def from_dict(cls, data, overrides=None):
            return cls()

    folder = _folder(tmp_path, "Toy-1B", model_type="toy_chat", chat_template=TEMPLATE)
    assert not is_instruct(folder) and build_prompter(folder) is None
    register_architecture("ToyChatLM", ToyConfig, lambda cfg: None, aliases=("toy_chat",), chat_by_default=True)
    register_architecture("ToyBaseLM", ToyConfig, lambda cfg: None, aliases=("toy_base",))
    try:
        assert is_instruct(folder) and build_prompter(folder).insert_prompt("x").endswith("<assistant>")
        assert not is_instruct(_folder(tmp_path, "Toy-1B-Base", model_type="toy_chat"))
        assert not is_instruct(_folder(tmp_path, "Other-1B", model_type="toy_base"))
        by_name = _folder(tmp_path, "Named-1B")
        (by_name / "config.json").write_text(json.dumps({"architectures": ["ToyChatLM"]}))
        assert is_instruct(by_name)
    finally:
        unregister_architecture("ToyChatLM")
        unregister_architecture("ToyBaseLM")
    assert not is_instruct(folder)


def test_templates_may_use_what_model_folders_templates_use():
    """Loop controls, a ``tojson`` that writes plain JSON (no HTML escapes, which would change the
    prompt's tokens; ``ensure_ascii`` and ``indent`` as arguments) and ``strftime_now``."""
    import datetime

    template = (
        "{% for m in messages %}{% if m['role'] == 'skip' %}{% continue %}{% endif %}"
        "{% if m['role'] == 'stop' %}{% break %}{% endif %}"
        "{{ m['content'] | tojson }};{% endfor %}"
        "{{ {'k': ['<a>', 'é']} | tojson(indent=1) }}|{{ 'é' | tojson(ensure_ascii=true) }}|{{ strftime_now('%Y') }}"
    )
    talk = [{"role": "user", "content": "<b> & \"q\" 'é'"}, {"role": "skip", "content": "no"},
            {"role": "user", "content": "two"}, {"role": "stop", "content": "x"}, {"role": "user", "content": "late"}]
    text = ChatPrompter(template).apply(talk)
    first, second, tail = text.split(";", 2)
    assert json.loads(first) == talk[0]["content"] and "<b> & " in first and "é" in first
    assert second == '"two"' and "late" not in text and '"no"' not in text
    indented, ascii_only, year = tail.split("|")
    assert indented == json.dumps({"k": ["<a>", "é"]}, ensure_ascii=False, indent=1)
    assert ascii_only == '"\\u00e9"' and year == str(datetime.datetime.now().year)
