"""A fake JNIEnv for driving the JNI symbols without a JVM: a function table with the slots the shims use at the
indices the JNI specification assigns them (6 FindClass, 14 ThrowNew, 17 ExceptionClear, 167 NewStringUTF,
179 NewIntArray, 200/203/204/205 Get{Byte,Int,Long,Float}ArrayRegion, 208/211/213 Set{Byte,Int,Float}ArrayRegion).
A Java array is modelled as an integer key into a dict of Python lists; a jstring as a key into a dict of strings."""
import ctypes

SLOT_COUNT = 235


class FakeEnv:
    def __init__(self, known_classes=("z/dragon/engine/cuda/impl/CudaException",)):
        self.arrays = {}
        self.thrown = []          # (class name, message)
        self.find_calls = []
        self.cleared = 0
        self.known = {name: 0x1000 + i for i, name in enumerate(known_classes)}
        self._rev = {v: k for k, v in self.known.items()}

        FIND = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        THROWNEW = ctypes.CFUNCTYPE(ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        CLEAR = ctypes.CFUNCTYPE(None, ctypes.c_void_p)
        GETLONG = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                                   ctypes.POINTER(ctypes.c_int64))

        def find(env, name):
            self.find_calls.append(name.decode())
            return self.known.get(name.decode(), None)

        def thrownew(env, cls, msg):
            self.thrown.append((self._rev.get(cls, "?"), msg.decode()))
            return 0

        def clear(env):
            self.cleared += 1

        def getlong(env, arr, start, n, buf):
            src = self.arrays[arr]
            for i in range(n):
                buf[i] = src[start + i]

        self.strings = {}

        def region_cb(ctype, to_java):
            proto = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctype))

            def get(env, arr, start, n, buf):      # Java array -> native buffer
                src = self.arrays[arr]
                for i in range(n):
                    buf[i] = src[start + i]

            def put(env, arr, start, n, buf):      # native buffer -> Java array
                dst = self.arrays[arr]
                for i in range(n):
                    dst[start + i] = buf[i]

            return proto(put if to_java else get)

        NEWSTR = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p)
        NEWINTS = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32)

        def newstr(env, utf):
            key = 0x3000 + len(self.strings)
            self.strings[key] = utf.decode()
            return key

        def newints(env, n):
            key = 0x2000 + len(self.arrays)
            self.arrays[key] = [0] * n
            return key

        extra = {167: NEWSTR(newstr), 179: NEWINTS(newints),
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

    def array(self, values):
        """A Java primitive array of any element type (byte[], int[], float[]); returns its handle."""
        key = 0x2000 + len(self.arrays)
        self.arrays[key] = list(values)
        return ctypes.c_void_p(key)

    def long_array(self, values):
        key = 0x2000 + len(self.arrays)
        self.arrays[key] = list(values)
        return ctypes.c_void_p(key)
