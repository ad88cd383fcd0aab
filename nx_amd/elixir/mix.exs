defmodule HipNx.MixProject do
  use Mix.Project

  # Needs a BEAM (Elixir >= 1.15) and ERTS headers; `make -C ../csrc` must have built
  # ../lib/libhipnx.so first.  The NIF shim is compiled by the :elixir_make compiler.
  def project do
    [
      app: :hipnx,
      version: "0.1.0",
      elixir: "~> 1.15",
      compilers: [:elixir_make] ++ Mix.compilers(),
      make_cwd: "c_src",
      deps: [{:nx, "~> 0.10"}, {:elixir_make, "~> 0.8", runtime: false}]
    ]
  end

  def application, do: [extra_applications: [:logger]]
end
