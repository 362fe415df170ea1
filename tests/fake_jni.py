"""A fake JNIEnv for driving the JNI symbols without a JVM: a function table with the slots the shims use at the
indices the JNI specification assigns them (6 FindClass, 14 ThrowNew, 17 ExceptionClear, 31 GetObjectClass, 94 GetFieldID,
104/105/109/110 Set{Object,Boolean,Int,Long}Field, 167 NewStringUTF, 176 NewByteArray, 179 NewIntArray,
200/203/204/205 Get{Byte,Int,Long,Float}ArrayRegion, 208/211/213 Set{Byte,Int,Float}ArrayRegion).
A Java array is modelled as an integer key into a dict of Python lists; a jstring as a key into a dict of strings; a Java
object (new_object) as a key into a dict of {field name: value} whose class declares a given set of (name, signature)
fields - GetFieldID returns NULL for a field the class does not declare, or declares with another signature, and
leaves an exception pending as a JVM does (so does FindClass for an unknown class). The JNI specification allows only
a handful of calls while an exception is pending (ExceptionClear among them): every other call made in that state is
recorded in `calls_while_pending`, which a correct shim leaves empty."""
import ctypes

SLOT_COUNT = 235


class FakeEnv:
    def __init__(self, known_classes=("z/dragon/engine/cuda/impl/CudaException",)):
        self.arrays = {}
        self.thrown = []          # (class name, message)
        self.find_calls = []
        self.cleared = 0
        self.pending = False              # an exception raised by a JNI call itself and not yet cleared
        self.calls_while_pending = []     # names of JNI calls the specification forbids in that state
        self.known = {name: 0x1000 + i for i, name in enumerate(known_classes)}
        self._rev = {v: k for k, v in self.known.items()}

        FIND = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        THROWNEW = ctypes.CFUNCTYPE(ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        CLEAR = ctypes.CFUNCTYPE(None, ctypes.c_void_p)
        GETLONG = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                                   ctypes.POINTER(ctypes.c_int64))

        def guard(what):
            if self.pending:
                self.calls_while_pending.append(what)

        def find(env, name):
            guard("FindClass")
            self.find_calls.append(name.decode())
            got = self.known.get(name.decode(), None)
            if got is None:
                self.pending = True       # NoClassDefFoundError
            return got

        def thrownew(env, cls, msg):
            guard("ThrowNew")
            self.thrown.append((self._rev.get(cls, "?"), msg.decode()))
            return 0

        def clear(env):
            self.cleared += 1
            self.pending = False

        def getlong(env, arr, start, n, buf):
            guard("GetLongArrayRegion")
            src = self.arrays[arr]
            for i in range(n):
                buf[i] = src[start + i]

        self.strings = {}

        def region_cb(ctype, to_java):
            proto = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctype))

            def get(env, arr, start, n, buf):      # Java array -> native buffer
                guard("GetArrayRegion")
                src = self.arrays[arr]
                for i in range(n):
                    buf[i] = src[start + i]

            def put(env, arr, start, n, buf):      # native buffer -> Java array
                guard("SetArrayRegion")
                dst = self.arrays[arr]
                for i in range(n):
                    dst[start + i] = buf[i]

            return proto(put if to_java else get)

        NEWSTR = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        NEWINTS = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32)

        def newstr(env, utf):
            guard("NewStringUTF")
            key = 0x3000 + len(self.strings)
            self.strings[key] = utf.decode()
            return key

        def newints(env, n):
            guard("NewIntArray")
            key = 0x2000 + len(self.arrays)
            self.arrays[key] = [0] * n
            return key

        # ---- objects and fields (CudaDevice.setProperty) ----
        self.objects = {}         # object handle -> {field name: value}
        self.declared = {}        # class handle -> {field name: signature}
        self.class_of = {}        # object handle -> class handle
        self.field_ids = {}       # field id -> (name, signature)
        self.set_calls = []       # (setter kind, field name) in call order
        V = ctypes.c_void_p
        GETCLS = ctypes.CFUNCTYPE(V, V, V)
        GETFID = ctypes.CFUNCTYPE(V, V, V, ctypes.c_char_p, ctypes.c_char_p)
        SETOBJ = ctypes.CFUNCTYPE(None, V, V, V, V)
        SETBOOL = ctypes.CFUNCTYPE(None, V, V, V, ctypes.c_uint8)
        SETINT = ctypes.CFUNCTYPE(None, V, V, V, ctypes.c_int32)
        SETLONG = ctypes.CFUNCTYPE(None, V, V, V, ctypes.c_int64)

        def getcls(env, obj):
            guard("GetObjectClass")
            return self.class_of[obj]

        def getfid(env, cls, name, sig):
            guard("GetFieldID")
            name, sig = name.decode(), sig.decode()
            if self.declared[cls].get(name) != sig:
                self.pending = True       # NoSuchFieldError
                return None
            fid = 0x5000 + len(self.field_ids)
            self.field_ids[fid] = (name, sig)
            return fid

        def setter(kind, expect):
            def put(env, obj, fid, value):
                guard("Set%sField" % kind)
                name, sig = self.field_ids[fid]
                assert sig in expect, "Set%sField on field %s of type %s" % (kind, name, sig)
                self.set_calls.append((kind, name))
                if kind == "Object":
                    value = self.strings[value] if value in self.strings else self.arrays[value]
                self.objects[obj][name] = bool(value) if kind == "Boolean" else value
            return put

        def newbytes(env, n):
            guard("NewByteArray")
            key = 0x2000 + len(self.arrays)
            self.arrays[key] = [0] * n
            return key

        extra = {31: GETCLS(getcls), 94: GETFID(getfid),
                 104: SETOBJ(setter("Object", ("Ljava/lang/String;", "[B", "[I"))), 105: SETBOOL(setter("Boolean", ("Z",))),
                 109: SETINT(setter("Int", ("I",))), 110: SETLONG(setter("Long", ("J",))), 176: NEWINTS(newbytes),
                 167: NEWSTR(newstr), 179: NEWINTS(newints),
                 200: region_cb(ctypes.c_int8, False), 203: region_cb(ctypes.c_int32, False), 205: region_cb(ctypes.c_float, False),
                 208: region_cb(ctypes.c_int8, True), 211: region_cb(ctypes.c_int32, True), 213: region_cb(ctypes.c_float, True)}
        self._cbs = (FIND(find), THROWNEW(thrownew), CLEAR(clear), GETLONG(getlong)) + tuple(extra.values())
        table = (ctypes.c_void_p * SLOT_COUNT)()
        table[6] = ctypes.cast(self._cbs[0], ctypes.c_void_p)
        table[14] = ctypes.cast(self._cbs[1], ctypes.c_void_p)
        table[17] = ctypes.cast(self._cbs[2], ctypes.c_void_p)
        table[204] = ctypes.cast(self._cbs[3], ctypes.c_void_p)
        for slot, cb in extra.items():
            table[slot] = ctypes.cast(cb, ctypes.c_void_p)
        self._table = table
        self._env = ctypes.c_void_p(ctypes.addressof(table))   # JNIEnv_ { const JNINativeInterface_* functions; }
        self.ptr = ctypes.pointer(self._env)

    def new_object(self, declared_fields):
        """A Java object whose class declares {field name: JNI signature}; returns its handle."""
        cls = 0x4000 + len(self.declared)
        self.declared[cls] = dict(declared_fields)
        obj = 0x6000 + len(self.objects)
        self.objects[obj] = {}
        self.class_of[obj] = cls
        return obj

    def array(self, values):
        """A Java primitive array of any element type (byte[], int[], float[]); returns its handle."""
        key = 0x2000 + len(self.arrays)
        self.arrays[key] = list(values)
        return ctypes.c_void_p(key)

    def long_array(self, values):
        key = 0x2000 + len(self.arrays)
        self.arrays[key] = list(values)
        return ctypes.c_void_p(key)
