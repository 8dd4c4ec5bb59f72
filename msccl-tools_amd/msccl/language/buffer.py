"""A named scratch buffer of one rank: grows as the program writes to it and is later given an
offset inside the rank's single scratch allocation (msccl/language/buffer.py)."""


class BufferSlice:
    def __init__(self, buf, name):
        self.name = name
        self.buf = buf
        self.offset = -1
        self.chunks = []

    def get_buffer(self):
        return self.buf

    def instance_size(self):
        return len(self.chunks)

    def set_offset(self, offset):
        self.offset = offset

    def get_global_index(self, index):
        assert self.offset > -1, "set_offset needs to be called first"
        return self.offset + index

    def __getitem__(self, index):
        return self.chunks[index]

    def __setitem__(self, index, value):
        if index >= len(self.chunks):
            self.chunks.extend([None] * (index + 1 - len(self.chunks)))
        self.chunks[index] = value

    def __len__(self):
        return len(self.chunks)
