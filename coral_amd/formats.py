"""Python view of the file-format entry points of libcoral_search.so (placeholder
until the C++ readers are registered)."""


def register(lib):
    return lib
