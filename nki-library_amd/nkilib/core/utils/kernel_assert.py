"""Argument validation helper with the reference's error text
(src/nkilib_src/nkilib/core/utils/kernel_assert.py:16-17)."""


def kernel_assert(condition: bool, error_text: str):
    if not condition:
        raise AssertionError(
            f"[INTERNAL_ERROR] [NCC_INKI016] Kernel validation exception: {error_text} - "
            "Please check the validation message and adjust kernel inputs accordingly"
        )


def assert_shape(tensor, expected_shape, tensor_name, error_text=""):
    kernel_assert(
        tuple(tensor.shape) == tuple(expected_shape),
        f"Received unexpected shape for {tensor_name}. "
        f"Expected {tuple(expected_shape)}, received {tuple(tensor.shape)}. {error_text}",
    )
