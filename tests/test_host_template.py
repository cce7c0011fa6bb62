"""The chat template engine (neura_amd/host/template.hpp, the mirror of crates/neura-template) against jinja2, the
published implementation of the language it reads a subset of: every rendering below is compared byte for byte with
jinja2's under its default environment (no block trimming, as the reference trims none).  The reference holds no test of
its own for this crate."""
import jinja2
import pytest

from neura_amd import host

QWEN = r'''{%- if tools %}
    {{- '<|im_start|>system\n' }}
    {%- if messages[0]['role'] == 'system' %}
        {{- messages[0]['content'] }}
    {%- else %}
        {{- 'You are Qwen, created by Alibaba Cloud. You are a helpful assistant.' }}
    {%- endif %}
    {{- "\n\n# Tools\n\nYou may call one or more functions to assist with the user query.\n\nYou are provided with function signatures within <tools></tools> XML tags:\n<tools>" }}
    {%- for tool in tools %}
        {{- "\n" }}
        {{- tool | tojson }}
    {%- endfor %}
    {{- "\n</tools>\n\nFor each function call, return a json object with function name and arguments within <tool_call></tool_call> XML tags:\n<tool_call>\n{\"name\": <function-name>, \"arguments\": <args-json-object>}\n</tool_call><|im_end|>\n" }}
{%- else %}
    {%- if messages[0]['role'] == 'system' %}
        {{- '<|im_start|>system\n' + messages[0]['content'] + '<|im_end|>\n' }}
    {%- else %}
        {{- '<|im_start|>system\nYou are Qwen, created by Alibaba Cloud. You are a helpful assistant.<|im_end|>\n' }}
    {%- endif %}
{%- endif %}
{%- for message in messages %}
    {%- if (message.role == "user") or (message.role == "system" and not loop.first) or (message.role == "assistant" and not message.tool_calls) %}
        {{- '<|im_start|>' + message.role + '\n' + message.content + '<|im_end|>' + '\n' }}
    {%- elif message.role == "assistant" %}
        {{- '<|im_start|>' + message.role }}
        {%- if message.content %}
            {{- '\n' + message.content }}
        {%- endif %}
        {%- for tool_call in message.tool_calls %}
            {%- if tool_call.function is defined %}
                {%- set tool_call = tool_call.function %}
            {%- endif %}
            {{- '\n<tool_call>\n{"name": "' }}
            {{- tool_call.name }}
            {{- '", "arguments": ' }}
            {{- tool_call.arguments | tojson }}
            {{- '}\n</tool_call>' }}
        {%- endfor %}
        {{- '<|im_end|>\n' }}
    {%- elif message.role == "tool" %}
        {%- if (loop.index0 == 0) or (messages[loop.index0 - 1].role != "tool") %}
            {{- '<|im_start|>user' }}
        {%- endif %}
        {{- '\n<tool_response>\n' }}
        {{- message.content }}
        {{- '\n</tool_response>' }}
        {%- if loop.last or (messages[loop.index0 + 1].role != "tool") %}
            {{- '<|im_end|>\n' }}
        {%- endif %}
    {%- endif %}
{%- endfor %}
{%- if add_generation_prompt %}
    {{- '<|im_start|>assistant\n' }}
{%- endif %}
'''

CHATML = "{% for message in messages %}{{'<|im_start|>' + message['role'] + '\n' + message['content'] + '<|im_end|>' + '\n'}}{% endfor %}{% if add_generation_prompt %}{{ '<|im_start|>assistant\n' }}{% endif %}"

TOOLS = [{"type": "function", "function": {"name": "weather", "description": "the <weather> & more in 'a' place",
                                           "parameters": {"type": "object", "properties": {"city": {"type": "string"}, "days": {"type": "integer"}},
                                                          "required": ["city"]}}}]
TALKS = [
    [{"role": "user", "content": "hello"}],
    [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hi\nthere"}, {"role": "assistant", "content": "yes?"},
     {"role": "user", "content": "größer 大きい 🙂"}],
    [{"role": "user", "content": "rain in Oslo?"},
     {"role": "assistant", "content": "", "tool_calls": [{"type": "function", "function": {"name": "weather", "arguments": {"city": "Oslo", "days": 2}}}]},
     {"role": "tool", "content": "{\"rain\": true}"}, {"role": "tool", "content": "{\"wind\": 3.5}"},
     {"role": "assistant", "content": "It rains."}, {"role": "system", "content": "a late system turn"}],
]


def jinja(source, messages, values):
    environment = jinja2.Environment(keep_trailing_newline=True)  # the reference drops no newline at the end of a template

    def raise_exception(text):
        raise RuntimeError(text)

    environment.globals["raise_exception"] = raise_exception
    return environment.from_string(source).render(messages=messages, **values)


@pytest.mark.parametrize("source", [QWEN, CHATML], ids=["qwen2.5", "chatml"])
@pytest.mark.parametrize("talk", range(len(TALKS)))
@pytest.mark.parametrize("prompt", [True, False])
@pytest.mark.parametrize("tools", [None, TOOLS], ids=["plain", "tools"])
def test_chat_templates_render_as_jinja2_renders_them(source, talk, prompt, tools):
    values = {"add_generation_prompt": prompt}
    if tools is not None:
        values["tools"] = tools
    assert host.render_template(source, TALKS[talk], values) == jinja(source, TALKS[talk], values)


PIECES = [
    # prints of every kind of value
    "{{ 1 }} {{ 2.5 }} {{ 3.0 }} {{ true }} {{ false }} {{ none }} {{ 'a' }} {{ missing }}|{{ items }} {{ table }} {{ 0.1 + 0.2 }} {{ -7 }} {{ - 2.5 }}",
    "{{ items[0] }} {{ items[-1] }} {{ items[1:] }} {{ items[:-1] }} {{ items[::2] }} {{ items[::-1] }} {{ items[3:0:-1] }} {{ items[-2:] }} {{ word[1] }} {{ word[-1] }}",
    "{{ table.b }} {{ table['c'] }} {{ table.nothing is defined }} {{ table['nothing'] is undefined }} {{ nested.inner.deep }}",
    # operators
    "{{ 1 + 2 }} {{ 5 - 7 }} {{ 1.5 + 1 }} {{ 'a' + 'b' }} {{ 'a' ~ 1 ~ 2.0 ~ true ~ none }} {{ 2 - 0.5 }}",
    "{{ 1 < 2 }} {{ 2 <= 2 }} {{ 3 > 4 }} {{ 4 >= 5 }} {{ 1 == 1.0 }} {{ 'a' != 'b' }} {{ 'a' < 'b' }} {{ items == items }} {{ none == none }} {{ 1 == '1' }}",
    "{{ 'ell' in word }} {{ 'z' not in word }} {{ 2 in items }} {{ 9 not in items }} {{ 'b' in table }} {{ 'q' in table }}",
    "{{ true and 'x' }} {{ false or 'y' }} {{ 0 or '' or 'z' }} {{ not 0 }} {{ not word }} {{ 1 and 0 }} {{ not 1 == 2 }} {{ (1 == 1) and (2 == 2) }}",
    "{{ 'yes' if items else 'no' }} {{ 'yes' if missing else 'no' }} {{ 1 if false else 2 if false else 3 }}",
    # filters and tests
    "[{{ '  pad  ' | trim }}] {{ items | length }} {{ word | length }} {{ table | length }} {{ 12 | string ~ 'x' }} {{ word | safe }} {{ items | tojson }} {{ table | tojson }}",
    "{{ special | tojson }} {{ nested | tojson }} {{ none | tojson }} {{ true | tojson }} {{ 1.5 | tojson }} {{ '' | tojson }}",
    "{{ word is string }} {{ 1 is number }} {{ 1.5 is number }} {{ 1 is integer }} {{ 1.5 is integer }} {{ true is boolean }} {{ none is none }} {{ 0 is none }}",
    "{{ items is iterable }} {{ word is iterable }} {{ table is mapping }} {{ items is mapping }} {{ items is sequence }} {{ true is true }} {{ false is false }} {{ 1 is not string }}",
    # statements
    "{% if items | length > 3 %}long{% elif items %}short{% else %}none{% endif %}|{% if missing %}a{% endif %}|{% if not missing %}b{% endif %}",
    "{% for item in items %}{{ loop.index }}/{{ loop.length }}:{{ item }}{% if not loop.last %}, {% endif %}{% endfor %}",
    "{% for item in items %}{{ loop.index0 }}{{ loop.first }}{{ loop.last }}{{ loop.previtem }}>{{ loop.nextitem }};{% endfor %}",
    "{% for key in table %}{{ key }}={{ table[key] }};{% endfor %}{% for letter in word %}<{{ letter }}>{% endfor %}{% for nothing in [] if false %}{% endfor %}"[:-len("{% for nothing in [] if false %}{% endfor %}")],
    "{% set total = 0 %}{% for item in items %}{% set total = total + item %}{% endfor %}{{ total }}",
    "{% set ns = namespace(total=0, seen='') %}{% for item in items %}{% set ns.total = ns.total + item %}{% set ns.seen = ns.seen ~ item %}{% endfor %}{{ ns.total }} {{ ns.seen }}",
    "{% macro greet(name, punctuation='!') %}Hello {{ name }}{{ punctuation }}{% endmacro %}{{ greet('a') }} {{ greet('b', '?') }} {{ greet(name='c', punctuation='.') }} {{ greet('d') | length }}",
    "{% macro wrap(text) %}[{{ text | trim }}]{% endmacro %}{% for item in items %}{{ wrap(' ' ~ item ~ ' ') }}{% endfor %}",
    # whitespace control and comments
    "a  {%- if true %}  b  {%- endif %}  c",
    "a  {% if true -%}  b  {% endif -%}  c {#- a comment -#}  d {# another #} e",
    "line\n  {{- 1 -}}  \n  next\n{%- for item in items -%}\n {{ item }}\n{%- endfor -%}\n end",
    # string methods and escapes
    "{{ 'a,b,,c'.split(',') }} {{ '  x '.strip() }}|{{ '  x '.lstrip() }}|{{ '  x '.rstrip() }}|{{ 'xxhixx'.strip('x') }} {{ word.startswith('he') }} {{ word.endswith('x') }}",
    "{{ 'tab\\there' }} {{ \"quote's\" }} {{ 'back\\\\slash' }} {{ 'new\\nline' }}",
    "{{ messages | length }} {{ messages[0].role }} {{ messages[-1]['content'] }} {% for m in messages %}{{ m.role[0] }}{% endfor %}",
]
VALUES = {"items": [1, 2, 3, 4, 5], "word": "hello", "table": {"b": 1, "c": "two", "a": [1.5, None, True]},
          "nested": {"inner": {"deep": "down", "z": 1}, "list": [{"k": "v"}, []]}, "special": "<a href=\"x\">it's & \\ \t\n é 🙂</a>"}


@pytest.mark.parametrize("piece", range(len(PIECES)))
def test_every_construct_renders_as_jinja2_renders_it(piece):
    source = PIECES[piece]
    assert host.render_template(source, TALKS[1], VALUES) == jinja(source, TALKS[1], VALUES)


def test_a_template_refuses_what_the_reference_refuses():
    for source, sentence in [
        ("{% block x %}{% endblock %}", "a template holds the block tag, and this renderer reads no such tag"),
        ("{{ 1 | upper }}", "the template filters a value through upper, and this renderer reads no such filter"),
        ("{{ 1 is odd }}", "the template weighs a value against the odd test, and this renderer reads no such test"),
        ("{{ 1", "a template opens a tag at byte 2 and holds no }} that closes it"),
        ("{% if true %}x", "a template ends where its elif or else or endif stands"),
        ("{{ raise_exception('roles must alternate') }}", "the template raises roles must alternate"),
        ("{{ items.nothing }}", "a template reads the attribute nothing of a list"),
        ("{{ items[9] }}", "a template reads the element 9 of a list of 5 elements"),
        ("{{ 1 + 'a' }}", "a template adds a string to a whole number"),
        ("{{ undefined_macro(1) }}", "a template calls undefined_macro, and this renderer reads no such macro or function"),
        ("{{ 'x' | trim(1) }}", "the template filters a value through the trim filter, and this renderer reads no argument of it"),
        ("{{ a ? b }}", "a tag of a template holds the character ? where this renderer reads no part of an expression"),
    ]:
        with pytest.raises(host.Panic) as refused:
            host.render_template(source, TALKS[0], VALUES)
        assert sentence in str(refused.value), (source, str(refused.value))


def test_a_gguf_carries_its_template(tmp_path):
    writer = host.Writer()
    writer.text("general.architecture", "qwen2")
    writer.text("tokenizer.chat_template", CHATML)
    writer.save(str(tmp_path / "t.gguf"))
    archive = host.GgufFile.open(tmp_path / "t.gguf")
    values = {"add_generation_prompt": True}
    assert host.render_template(archive, TALKS[1], values) == jinja(CHATML, TALKS[1], values)
    archive.close()
    writer = host.Writer()
    writer.text("general.architecture", "qwen2")
    writer.save(str(tmp_path / "none.gguf"))
    archive = host.GgufFile.open(tmp_path / "none.gguf")
    with pytest.raises(host.Panic, match="tokenizer.chat_template"):
        host.render_template(archive, TALKS[0])
    archive.close()
