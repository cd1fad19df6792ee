"""Chat templates (host logic, no GPU): `ChatTemplate::apply` of the reference's chat front end
(crates/wgml-chat/src/chat_template.rs:27-39) renders `tokenizer.chat_template`, or the Llama-2
default (models/llama2/llama-2-chat.jinja), with minijinja (`trim_blocks` on; globals bos_token,
eos_token, add_generation_prompt = true).  The engine is not available offline and the reference
holds no rendered output, so the expected strings below are traced by hand from the template
text and the template language's published rules: which branches run, what the expressions
give, and which line breaks and indentation between the blocks survive `trim_blocks` (the first
newline after a block tag is dropped, nothing else).  Rendering of a real model's template by
the real engine: parity unpinned."""
import pytest

from wgml_amd.chat_template import LLAMA2_CHAT_TEMPLATE, ChatTemplate, Prompt, TemplateError
from wgml_amd.tokenizer import llama2_chat_prompt

def test_default_template_single_user_turn_exact_whitespace():
    # else-branch of the system test, one loop iteration, user branch.  Pieces, in order:
    #   "    " before {% set system_message = '' %} (its newline dropped), "\n" (the empty line 7),
    #   "    " before the alternation test, "\n" (line 12), "    " before `if loop.index0 == 0`,
    #   "        " before the set of its true branch, "    " before {% else %}, "\n" (line 18),
    #   "    " before the role test, "        " + the user text + "\n" (a newline after {{ }} stays),
    #   "    " before {% elif %}; nothing after {% endif %} / {% endfor %}
    out = ChatTemplate(LLAMA2_CHAT_TEMPLATE).apply([{"role": "user", "content": "  Hi there \n"}], "<s>", "</s>")
    want = "    \n" + "    " + "\n" + "    " + "        " + "    " + "\n" + "    " + "        " + \
           "<s>[INST] Hi there [/INST]" + "\n" + "    "
    assert out == want


def test_default_template_system_message_and_three_turns():
    # system message folded into the first user turn; user / assistant / user.  The values the
    # branches emit are what llama2_chat_prompt builds directly; between them sits the
    # whitespace of the template's layout: "    " twice (the two set statements of the system
    # branch) and the empty line 7 in front, and around every value the same pieces as in the
    # single-turn case (both branches of `if loop.index0 == 0` leave "        " + "    ").
    msgs = [{"role": "system", "content": " Be brief. "}, {"role": "user", "content": "What is 2+2?"},
            {"role": "assistant", "content": "4"}, {"role": "user", "content": "And 3+3?\n"}]
    values = ["<s>[INST] <<SYS>>\nBe brief.\n<</SYS>>\n\nWhat is 2+2? [/INST]", " 4 </s>",
              "<s>[INST] And 3+3? [/INST]"]
    assert "".join(values) == llama2_chat_prompt(msgs, "<s>", "</s>")

    def turn(value):
        return "    " + "\n" + "    " + "        " + "    " + "\n" + "    " + "        " + value + "\n" + "    "

    want = "    " + "    " + "\n" + "".join(turn(v) for v in values)
    assert ChatTemplate(LLAMA2_CHAT_TEMPLATE).apply(msgs, "<s>", "</s>") == want


def test_default_template_filter_binds_tighter_than_plus():
    # `bos_token + '[INST] ' + content | trim + ' [/INST]'` trims content only: the space before
    # [/INST] and after [INST] stay
    out = ChatTemplate("{% set a = 'A' %}{% set b = '  B  ' %}{{ a + ' x ' + b | trim + ' y ' }}").apply([], "", "")
    assert out == "A x B y "


def test_roles_must_alternate():
    t = ChatTemplate(LLAMA2_CHAT_TEMPLATE)
    with pytest.raises(TemplateError, match="alternate"):
        t.apply([{"role": "assistant", "content": "x"}], "<s>", "</s>")
    with pytest.raises(TemplateError, match="alternate"):
        t.apply([{"role": "user", "content": "a"}, {"role": "user", "content": "b"}], "<s>", "</s>")


CHATML = ("{% for message in messages %}{{'<|im_start|>' + message['role'] + '\\n' + message['content'] + "
          "'<|im_end|>' + '\\n'}}{% endfor %}{% if add_generation_prompt %}{{ '<|im_start|>assistant\\n' }}{% endif %}")


def test_chatml_template():
    p = Prompt().append_system("You are helpful.").append_user("Hello").append_assistant("Hi!").append_user("Bye")
    out = ChatTemplate(CHATML).apply(p, "<s>", "</s>")
    assert out == ("<|im_start|>system\nYou are helpful.<|im_end|>\n<|im_start|>user\nHello<|im_end|>\n"
                   "<|im_start|>assistant\nHi!<|im_end|>\n<|im_start|>user\nBye<|im_end|>\n<|im_start|>assistant\n")
    assert ChatTemplate(CHATML).apply(p, "", "", add_generation_prompt=False).endswith("Bye<|im_end|>\n")


LLAMA3 = ("{% set loop_messages = messages %}{% for message in loop_messages %}"
          "{% set content = '<|start_header_id|>' + message['role'] + '<|end_header_id|>\\n\\n'+ message['content'] | trim + '<|eot_id|>' %}"
          "{% if loop.index0 == 0 %}{% set content = bos_token + content %}{% endif %}{{ content }}{% endfor %}"
          "{% if add_generation_prompt %}{{ '<|start_header_id|>assistant<|end_header_id|>\\n\\n' }}{% endif %}")


def test_llama3_style_template():
    out = ChatTemplate(LLAMA3).apply([{"role": "system", "content": "S "}, {"role": "user", "content": " U"}],
                                     "<|begin_of_text|>", "<|end_of_text|>")
    assert out == ("<|begin_of_text|><|start_header_id|>system<|end_header_id|>\n\nS<|eot_id|>"
                   "<|start_header_id|>user<|end_header_id|>\n\nU<|eot_id|>"
                   "<|start_header_id|>assistant<|end_header_id|>\n\n")


def test_whitespace_control_and_trim_blocks():
    # `-` strips the neighbouring text; trim_blocks drops one newline after a block tag only
    t = "a  {%- if true %}\n  b\n{% endif -%}  \n c{{ 1 }}\n{{- 2 }}\n"
    assert ChatTemplate(t).apply([], "", "") == "a  b\nc12\n"
    assert ChatTemplate("{# note #}\nx").apply([], "", "") == "x"
    assert ChatTemplate("{{ 'v' }}\nx").apply([], "", "") == "v\nx"


def test_expressions():
    def r(src, **kw):
        return ChatTemplate(src).apply(kw.get("messages", []), "B", "E")
    assert r("{{ 7 % 4 }}|{{ 7 // 2 }}|{{ 2 * 3 + 1 }}|{{ 'a' ~ 1 ~ 'b' }}") == "3|3|7|a1b"
    assert r("{{ 'x' if 1 > 2 else 'y' }}{{ 'z' if false }}") == "y"
    assert r("{{ [1, 2, 3] | last }}{{ [1, 2, 3][-1] }}{{ [1, 2, 3][1:] | length }}{{ 'a,b'.split(',') | first }}") == "332a"
    assert r("{{ ' pad ' | trim | upper }}{{ undefined_name | default('d') }}{{ 'a b' | split(' ') | join('-') }}") == "PADda-b"
    assert r("{% if x is defined %}1{% else %}0{% endif %}{% if bos_token is string and eos_token == 'E' %}1{% endif %}") == "01"
    assert r("{% if 'b' in 'abc' and 'z' not in 'abc' and not false %}ok{% endif %}") == "ok"
    msgs = [{"role": "user", "content": "q"}, {"role": "assistant", "content": "a"}]
    assert r("{% for m in messages %}{{ loop.index }}{{ m.role[0] }}{% if not loop.last %},{% endif %}{% endfor %}",
             messages=msgs) == "1u,2a"
    # a loop body is a scope of its own; a namespace carries a value out of it
    assert r("{% set n = 0 %}{% for m in messages %}{% set n = n + 1 %}{% endfor %}{{ n }}", messages=msgs) == "0"
    assert r("{% set ns = namespace(n=0) %}{% for m in messages %}{% set ns.n = ns.n + 1 %}{% endfor %}{{ ns.n }}",
             messages=msgs) == "2"
    assert r("{{ messages[5]['role'] }}|{{ messages | length }}") == "|0"
    with pytest.raises(TemplateError):
        ChatTemplate("{% if x %}")
    with pytest.raises(TemplateError):
        ChatTemplate("{{ 1 + }}").apply([], "", "")
    with pytest.raises(TemplateError):
        ChatTemplate("{% frobnicate %}")


def test_from_gguf_falls_back_to_the_default():
    class G:
        metadata = {}
    assert ChatTemplate.from_gguf(G()).template == LLAMA2_CHAT_TEMPLATE
    G.metadata = {"tokenizer.chat_template": CHATML}
    assert ChatTemplate.from_gguf(G()).template == CHATML
