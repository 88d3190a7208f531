"""Test and benchmark harness, not product: what records the graphs the reference's front end would hand to the backend
(lazy tensor ops and the tape's gradient rules, the resnet-train model, a handful of front-end lowerings) and the script
that measures fusion plans for the cost-model fit. The backend (helium_amd/) depends on none of it."""
