"""The reference's NetDef schema (blaze/proto/blaze.proto:6-115) as dynamic protobuf classes.

Test helper: the image has the protobuf python runtime but no protoc, so the descriptors are built by hand
(field names, numbers, labels and types as in the .proto).  Gives the tests an independent implementation of
both protobuf encodings to hold the C++ text/wire readers against.
"""
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

_F = descriptor_pb2.FieldDescriptorProto
_OPT, _REQ, _REP = _F.LABEL_OPTIONAL, _F.LABEL_REQUIRED, _F.LABEL_REPEATED


def _field(msg, name, number, ftype, label=_OPT, type_name=None, packed=False, default=None):
    f = msg.field.add()
    f.name, f.number, f.type, f.label = name, number, ftype, label
    if type_name:
        f.type_name = type_name
    if packed:
        f.options.packed = True
    if default is not None:
        f.default_value = default


def _build():
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name = "blaze_test.proto"
    fd.package = "blaze"
    fd.syntax = "proto2"
    m = fd.message_type.add()
    m.name = "TensorShape"
    _field(m, "dims", 1, _F.TYPE_INT64, _REP)
    m = fd.message_type.add()
    m.name = "Argument"
    _field(m, "name", 1, _F.TYPE_STRING)
    _field(m, "f", 2, _F.TYPE_FLOAT)
    _field(m, "i", 3, _F.TYPE_INT64)
    _field(m, "s", 4, _F.TYPE_BYTES)
    _field(m, "floats", 5, _F.TYPE_FLOAT, _REP, packed=True)
    _field(m, "ints", 6, _F.TYPE_INT64, _REP, packed=True)
    _field(m, "strings", 7, _F.TYPE_BYTES, _REP)
    m = fd.message_type.add()
    m.name = "DeviceOption"
    _field(m, "device_type", 1, _F.TYPE_INT32, default="0")
    _field(m, "device_id", 2, _F.TYPE_INT32, default="0")
    _field(m, "is_pipe", 3, _F.TYPE_BOOL, default="false")
    m = fd.message_type.add()
    m.name = "OperatorDef"
    _field(m, "type", 1, _F.TYPE_STRING, _REQ)
    _field(m, "name", 2, _F.TYPE_STRING)
    _field(m, "input", 3, _F.TYPE_STRING, _REP)
    _field(m, "output", 4, _F.TYPE_STRING, _REP)
    _field(m, "arg", 5, _F.TYPE_MESSAGE, _REP, ".blaze.Argument")
    _field(m, "device_option", 6, _F.TYPE_MESSAGE, _OPT, ".blaze.DeviceOption")
    _field(m, "doc_string", 7, _F.TYPE_STRING)
    m = fd.message_type.add()
    m.name = "ValueInfo"
    _field(m, "name", 1, _F.TYPE_STRING)
    _field(m, "dtype", 2, _F.TYPE_INT32)  # enum DataType on the wire = varint
    _field(m, "doc_string", 3, _F.TYPE_STRING)
    _field(m, "level", 4, _F.TYPE_INT32, default="0")
    _field(m, "input_type", 5, _F.TYPE_INT32)
    _field(m, "feature_name", 6, _F.TYPE_STRING)
    _field(m, "tensor_shape", 7, _F.TYPE_MESSAGE, _OPT, ".blaze.TensorShape")
    m = fd.message_type.add()
    m.name = "NetDef"
    _field(m, "name", 1, _F.TYPE_STRING)
    _field(m, "op", 2, _F.TYPE_MESSAGE, _REP, ".blaze.OperatorDef")
    _field(m, "run_mode", 3, _F.TYPE_STRING, default="simple")
    _field(m, "arg", 4, _F.TYPE_MESSAGE, _REP, ".blaze.Argument")
    _field(m, "device_option", 5, _F.TYPE_MESSAGE, _OPT, ".blaze.DeviceOption")
    _field(m, "external_input", 6, _F.TYPE_MESSAGE, _REP, ".blaze.ValueInfo")
    _field(m, "external_output", 7, _F.TYPE_MESSAGE, _REP, ".blaze.ValueInfo")
    _field(m, "model_str", 8, _F.TYPE_BYTES)
    _field(m, "version", 9, _F.TYPE_INT32, default="1000")
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    if get is None:
        factory = message_factory.MessageFactory(pool)
        return {n: factory.GetPrototype(pool.FindMessageTypeByName("blaze." + n)) for n in ("NetDef", "OperatorDef", "Argument")}
    return {n: get(pool.FindMessageTypeByName("blaze." + n)) for n in ("NetDef", "OperatorDef", "Argument")}


CLASSES = _build()
NetDef = CLASSES["NetDef"]
