"""The text-format reader (deepnet_amd/pbtxt.py) that stands in for protobuf's text_format on
deepnet's model / operation files: grammar cases written out by hand, the "fields that are
set win" merge of deepnet/neuralnet.py:78-93, and the model files under tests/golden/ (written
for these tests in the format of deepnet/examples/*/model*.pbtxt)."""
import os

import pytest

from deepnet_amd import pbtxt

HERE = os.path.dirname(os.path.abspath(__file__))


def test_scalars_messages_comments_and_repeats():
    m = pbtxt.parse('''
      # a comment
      name: "a \\"quoted\\" name"   'and more'
      count: 3 ratio : -0.5e-1 big: 1e3 flag: true other: false kind: DENSE_GAUSSIAN
      shape: 28 shape: 28
      shape: 1     # trailing comment
      dims: [2, 3]
      sub { x: 1 inner < y: 2.5f > }
      sub: { x: 2; }
    ''')
    assert m.name == 'a "quoted" name' 'and more'
    assert m.count == 3 and isinstance(m.count, int)
    assert m.ratio == -0.05 and m.big == 1000.0 and isinstance(m.big, float)
    assert m.flag is True and m.other is False and m.kind == 'DENSE_GAUSSIAN'
    assert m.all('shape') == [28, 28, 1] and m.all('dims') == [2, 3]
    subs = m.all('sub')
    assert [s.x for s in subs] == [1, 2] and subs[0].inner.y == 2.5
    assert m.get('sub') is subs[1]                       # a non-repeated read sees the last one
    assert 'missing' not in m and m.get('missing', 7) == 7
    with pytest.raises(AttributeError):
        m.missing
    assert m.names() == ['name', 'count', 'ratio', 'big', 'flag', 'other', 'kind', 'shape', 'dims', 'sub']


@pytest.mark.parametrize("text", ['a: ', 'a { b: 1', 'a b', ': 3', 'a: 1 }', 'a: "unterminated', 'a: 1 $'])
def test_malformed_text_is_refused(text):
    with pytest.raises(pbtxt.ParseError):
        pbtxt.parse(text)


def test_merge_keeps_unset_fields_and_overwrites_set_ones():
    base = pbtxt.parse('base_epsilon: 0.1 apply_l2_decay: true l2_decay: 0.001 activation: LOGISTIC')
    over = pbtxt.parse('apply_l2_decay: false dropout: true')
    got = pbtxt.merged(base, over).scalars()
    assert got == dict(base_epsilon=0.1, apply_l2_decay=False, l2_decay=0.001, activation='LOGISTIC', dropout=True)
    assert pbtxt.merged(None, over).scalars() == over.scalars()
    assert pbtxt.merged(base, None).scalars() == base.scalars()
    nested = pbtxt.merged(pbtxt.parse('a { x: 1 y: 2 }'), pbtxt.parse('a { y: 3 } b: 4'))
    assert nested.a.scalars() == dict(x=1, y=3) and nested.b == 4


def test_model_files_of_the_tests():
    m = pbtxt.parse(open(os.path.join(HERE, 'golden', 'small_convnet.pbtxt')).read())
    assert m.model_type == 'FEED_FORWARD_NET' and m.seed == 17
    assert [l.name for l in m.all('layer')] == ['input_layer', 'output_layer', 'hidden1', 'hidden2', 'hidden3']
    assert m.all('layer')[0].all('shape') == [12, 12, 2]
    e = m.all('edge')[0]
    cv = e.param.conv_params
    assert e.param.conv is True and (cv.size, cv.num_filters, cv.pool_stride, cv.rnorm) == (3, 16, 2, True)
    assert e.hyperparams.initial_momentum == 0.9
    r = pbtxt.parse(open(os.path.join(HERE, 'golden', 'small_rbm.pbtxt')).read())
    assert r.model_type == 'DBM' and r.all('edge')[0].directed is False
    assert r.all('layer')[1].hyperparams.sparsity is True


def test_read_model_takes_text_files_only(tmp_path):
    from deepnet_amd import util
    p = tmp_path / 'op.pbtxt'
    p.write_text('optimizer: CD\nstopcondition { steps: 10 }\nbatchsize: 32\n')
    op = util.ReadOperation(str(p))
    assert op.optimizer == 'CD' and op.stopcondition.steps == 10 and op.batchsize == 32
    with pytest.raises(NotImplementedError):
        util.ReadModel(str(tmp_path / 'model.gz'))


def test_written_text_reads_back_the_same_tree():
    m = pbtxt.parse(open(os.path.join(HERE, 'golden', 'small_convnet.pbtxt')).read())
    assert pbtxt.parse(pbtxt.dumps(m)) == m
    extra = pbtxt.Message()
    extra.add('mat', bytes(range(256)))
    extra.add('text', 'a "quoted" \\ back\nslash')
    extra.add('tiny', 1e-30)
    extra.add('kind', pbtxt.Enum('PCD'))
    text = pbtxt.dumps(extra)
    assert all(32 <= ord(c) < 127 or c == '\n' for c in text)            # printable ASCII: octal escapes for the rest
    back = pbtxt.parse(text)
    assert back.mat.encode('latin-1') == bytes(range(256))
    assert back.text == 'a "quoted" \\ back\nslash' and back.tiny == 1e-30
    assert back.kind == 'PCD' and isinstance(back.kind, pbtxt.Enum) and 'kind: PCD' in text
    m.set('seed', 3)
    m.set('shape', 1, 2)
    assert m.seed == 3 and m.names().index('seed') == 2 and m.all('shape') == [1, 2]


def test_bytes_fields_survive_parse_and_dumps_more_than_once(tmp_path):
    """A stored parameter is raw float32 bytes (util.py:13-21); most of them are >= 0x80.  A
    parsed model holds them as a str with one character per byte, and writing that back must
    give the same bytes again, however often."""
    import numpy as np
    from deepnet_amd import util
    arr = np.array([[-1.5, 3.25e-7], [1e30, -0.0]], dtype=np.float32)
    raw = arr.tobytes() + bytes(range(256))
    m = pbtxt.Message()
    p = pbtxt.Message()
    p.add('name', 'weight')
    p.add('mat', raw)
    m.add('param', p)
    text1 = pbtxt.dumps(m)
    once = pbtxt.parse(text1)
    text2 = pbtxt.dumps(once)
    twice = pbtxt.parse(text2)
    assert text1 == text2 and text1.isascii()
    for got in (once.param.mat, twice.param.mat):
        assert len(got) == len(raw) and got.encode('latin-1') == raw
    # ReadModel -> WritePbtxt -> ReadModel
    path1, path2 = str(tmp_path / 'a.pbtxt'), str(tmp_path / 'b.pbtxt')
    util.WritePbtxt(path1, m)
    util.WritePbtxt(path2, util.ReadModel(path1))
    assert util.ReadModel(path2).param.mat.encode('latin-1') == raw
    # text beyond latin-1 is still written (as UTF-8 bytes)
    assert '\\' in pbtxt.dumps(pbtxt.parse('name: "\u4e2d"'))


def test_octal_and_hex_escapes_of_one_to_three_digits():
    m = pbtxt.parse(r'a: "\0" b: "\18" c: "\101\7z" d: "\x41\377" e: "\1019"')
    assert m.a == '\x00' and m.b == '\x018' and m.c == 'A\x07z' and m.d == 'A\xff' and m.e == 'A9'
